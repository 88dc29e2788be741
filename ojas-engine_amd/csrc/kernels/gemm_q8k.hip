// Family "gemm_q8k": Q4_K rows against a batch of tokens on the int8 matrix cores, in the CPU
// reference's arithmetic — activations quantized per 256 by quant_q8k, integer dots per 32-weight
// sub-block, the scale algebra of dot_q4k (crates/ojas-cpu/src/cpu_math.rs:539-635):
//     y[t][n] (=, +=) sum_sb sx[t][sb] * ( d * sum_j sc_j * idot_j  -  dmin * sum_j m_j * bsum_j ).
// This is what serves speculative verify (2-16 tokens on every projection) and prefill chunks
// with results within the parity bar of the CPU path, which an f16 tile cannot give.
//
//   gemm_q8k_q4k_mf(xq, xs, w, y, K, N, M, ACC, RW, RT)   block 256, grid [x <= ceil(N / (16 RW RT)), ceil(M / 64), 1]
//
// v_mfma_i32_16x16x32_i8 multiplies 16 tokens x 16 rows over one sub-block:
//   A: lane (m, kg) = (lane % 16, lane / 16) holds int8 positions 8 kg .. 8 kg + 7 of token m;
//   B: lane (n, kg) the 4-bit codes of the same positions of row n, as bytes;
//   D: register v of lane (n, kg) = idot of token 4 kg + v with row n.
// The row is lane-constant in D, so a sub-block's 6-bit scale enters with one v_mad_i32_i24 per D
// register (the sum over the eight sub-blocks is exact in int32).  The min term
// sum_j m_j * bsum_j is itself a small product over j: the workgroup splits every bsum (|.| <= 4064)
// into 64 hi + lo with both parts in int8 while it stages the tokens, and two more MFMAs per
// super-block (the row's eight mins as B in the first eight positions) give sum_j m_j lo_j and
// sum_j m_j hi_j for all 16 x 16 outputs at once.  A super-block ends with two converts and
// three FMAs per output.
//
// A workgroup owns 16 RW RT rows (RW = 1, 2 or 4 row tiles side by side, each wave RT of them one after
// the other per staged chunk; only RT = 1 is built) and up to 64 tokens (P = 1, 2 or 4 passes of
// 16; eight passes do not fit the register file); its four waves are RW row tiles x KW = 4 / RW slices of the super-blocks.  Tokens wait in
// LDS, chunk by chunk of K (as many super-blocks as fit 76 KB for the workgroup's tokens: 256 bytes,
// a scale and 16 bytes of split sums per token and super-block), rows 32 bytes longer than the
// chunk so that an 8-byte read of 64 lanes spreads over all banks.
// K-slices meet in LDS in wave order.
#include "ojk_common.h"
#include "ojk_gq.h"

#define GQ_LDS 77824u

template <int P, int RT>
__device__ __forceinline__ void gemm_q8k_q4k_mf_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                                     const uchar* __restrict__ w, float* __restrict__ y,
                                                     uint K, uint N, uint M, uint ACC, uint RW, uchar* lds) {
    const uint tid = threadIdx.x, lane = tid & 63u;
    const uint wave = (uint)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint nsb = K >> 8, KW = 4u / RW, rt = wave / KW, kw = wave % KW;
    const uint BM = 16u * P, t0 = blockIdx.y * 64u;
    // LDS: [reduction buffer: 4 waves x RT x P x 4 x 64 floats] [tokens] [token scales] [split bsums].
    // Chunk of K staged at a time: BM * (KC + 32) + (KC / 256) * BM * 20 bytes, a whole multiple of
    // KW super-blocks so that a wave's slice continues from chunk to chunk (the host picks RW so
    // that at least KW fit).  When the whole K fits, the tokens are staged once and the workgroup
    // walks row groups blockIdx.x, blockIdx.x + gridDim.x, ...
    float* red = (float*)lds;
    uchar* tok = lds + 4096u * P * (KW > 1u ? RT : 0u);
    const uint fit = ((GQ_LDS - 4096u * P * (KW > 1u ? RT : 0u)) / BM - 32u) / 276u;
    const bool whole = nsb <= fit;
    const uint csb = whole ? nsb : fit / KW * KW;                // super-blocks per chunk
    const uint S = csb * 256u + 32u;
    float* lsx = (float*)(tok + (size_t)BM * S);                 // [csb][BM] token scales
    uchar* lbq = (uchar*)(lsx + csb * BM);                       // [csb][BM][16]: lo_0..7, hi_0..7 of the bsums
    const uint n = lane & 15u, kg = lane >> 4;
    const uchar* xa = tok + (size_t)n * S + 8u * kg;
    const gq_i4 zero = {0, 0, 0, 0};
    const uint ngroups = (N + 16u * RW * RT - 1u) / (16u * RW * RT);
    const size_t rtb = (size_t)16u * RW * nsb * Q4K_BYTES;       // bytes from a row tile of this wave to its next
    for (uint grp = blockIdx.x; grp < ngroups; grp += gridDim.x) {
        // this wave's row tiles: (grp * RT + q) * RW + rt, q = 0 .. RT - 1 (rows past N clamped per tile)
        const uint tile0 = grp * RT * RW + rt;
        uint rowq[RT];
#pragma unroll
        for (int q = 0; q < RT; q++) rowq[q] = min((tile0 + (uint)q * RW) * 16u + n, N - 1u);
        float acc[RT][P][4];
#pragma unroll
        for (int q = 0; q < RT; q++)
#pragma unroll
            for (int p = 0; p < P; p++)
#pragma unroll
                for (int v = 0; v < 4; v++) acc[q][p][v] = 0.0f;
        GqW cur = gq_load(w + ((size_t)rowq[0] * nsb + min(kw, nsb - 1u)) * Q4K_BYTES, kg);
        for (uint sb0 = 0; sb0 < nsb; sb0 += csb) {
            const uint cn = min(csb, nsb - sb0);                 // super-blocks in this chunk
            if (!whole || grp == blockIdx.x) {
                if (sb0 || grp != blockIdx.x) __syncthreads();   // everyone is done with the previous chunk
                // stage tokens t0 .. t0 + BM - 1 (zeros past M): a thread keeps one 16-byte column of the
                // chunk and walks the tokens eight loads at a time (one wait per eight, not per load)
                const uint per_row = cn * 16u, lpr = min(per_row, 256u), rpp = 256u / lpr;
                const uint c0 = tid % lpr, ts = tid / lpr;
                if (ts < rpp) {
                    for (uint c = c0; c < per_row; c += lpr) {
                        const signed char* src = xq + (size_t)t0 * K + (size_t)sb0 * 256u + (size_t)c * 16u;
                        for (uint tb = ts; tb < BM; tb += 8u * rpp) {
                            uint4 v[8];
#pragma unroll
                            for (int u = 0; u < 8; u++) {
                                const uint t = tb + (uint)u * rpp;
                                v[u] = make_uint4(0u, 0u, 0u, 0u);
                                if (t < BM && t0 + t < M) v[u] = *(const uint4*)(src + (size_t)t * K);
                            }
#pragma unroll
                            for (int u = 0; u < 8; u++) {
                                const uint t = tb + (uint)u * rpp;
                                if (t < BM) *(uint4*)(tok + (size_t)t * S + (size_t)c * 16u) = v[u];
                            }
                        }
                    }
                }
                for (uint i = tid; i < cn * BM; i += 256u) {
                    const uint s = i / BM, t = i - s * BM;
                    lsx[i] = t0 + t < M ? xs[(size_t)(t0 + t) * nsb + sb0 + s] : 0.0f;
                }
                __syncthreads();
                // bsum of every (token, sub-block) of the chunk, split into int8 parts: 64 * hi + lo
                for (uint i = tid; i < cn * BM * 8u; i += 256u) {
                    const uint jj = i & 7u, t = (i >> 3) % BM, s = i / (8u * BM);
                    const uint4* px = (const uint4*)(tok + (size_t)t * S + s * 256u + jj * 32u);
                    const uint4 a = px[0], b = px[1];
                    int bs = dot4_i8(a.x, 0x01010101u, 0);
                    bs = dot4_i8(a.y, 0x01010101u, bs); bs = dot4_i8(a.z, 0x01010101u, bs); bs = dot4_i8(a.w, 0x01010101u, bs);
                    bs = dot4_i8(b.x, 0x01010101u, bs); bs = dot4_i8(b.y, 0x01010101u, bs);
                    bs = dot4_i8(b.z, 0x01010101u, bs); bs = dot4_i8(b.w, 0x01010101u, bs);
                    uchar* o = lbq + ((size_t)s * BM + t) * 16u;
                    o[jj] = (uchar)(bs & 63);
                    o[8u + jj] = (uchar)(bs >> 6);
                }
                __syncthreads();
            }
            for (uint s = kw; s < cn; s += KW) {
                const uint nxt = s + KW < cn ? sb0 + s + KW : sb0 + csb + kw;   // this slice's next super-block
#pragma unroll
                for (int q = 0; q < RT; q++) {
                    // the next (row tile, super-block) of this wave is on its way
                    const GqW nx = q + 1 < RT
                        ? gq_load(w + ((size_t)rowq[q + 1 < RT ? q + 1 : 0] * nsb + sb0 + s) * Q4K_BYTES, kg)
                        : gq_load(w + ((size_t)rowq[0] * nsb + min(nxt, nsb - 1u)) * Q4K_BYTES, kg);
                    const float d = f16_bits_to_f32(cur.hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(cur.hdr.x >> 16);
                    // all eight scales and mins at once, a byte each (as in gq_superblock)
                    const uint sc_lo = cur.hdr.y & 0x3F3F3F3Fu, mn_lo = cur.hdr.z & 0x3F3F3F3Fu;
                    const uint sc_hi = (cur.hdr.w & 0x0F0F0F0Fu) | ((cur.hdr.y >> 2) & 0x30303030u);
                    const uint mn_hi = ((cur.hdr.w >> 4) & 0x0F0F0F0Fu) | ((cur.hdr.z >> 2) & 0x30303030u);
                    const long Bm = kg == 0u ? gq_pack(mn_lo, mn_hi) : 0;    // only positions 0..7 carry mins
                    if (P >= 2) {
                        // Several passes share the row tile: fold the 6-bit scales into the codes once instead of
                        // into every result.  sc = 8 sh + sl with sl, sh <= 7, so sl * q and sh * q (<= 105) are
                        // int8 again and a packed 16-bit multiply scales four codes at once without a carry between
                        // bytes; two accumulating MFMAs per sub-block then give  sum_j sl_j idot_j  and
                        // sum_j sh_j idot_j, and  sum_j sc_j idot_j = 8 * (the second) + (the first)  exactly.
                        // One v_mfma_i32_16x16x64_i8 then covers a whole 64-weight chunk — its low-nibble
                        // sub-block in positions 0..7 of the lane's sixteen, its high-nibble sub-block in positions
                        // 8..15, each under its own folded scale — against the lane's 8 + 8 activations of the two
                        // sub-blocks (what matters is that A and B put the same weight position in the same slot).
                        gq_i4 BA[4], BB[4];
#pragma unroll
                        for (int c = 0; c < 4; c++) {
                            // chunk c = sub-blocks 2c (low nibbles) and 2c + 1 (high nibbles)
                            const uint se = 2 * c < 4 ? (sc_lo >> (16 * c)) & 0xFFu : (sc_hi >> (16 * (c - 2))) & 0xFFu;
                            const uint so = 2 * c < 4 ? (sc_lo >> (16 * c + 8)) & 0xFFu : (sc_hi >> (16 * (c - 2) + 8)) & 0xFFu;
                            const gq_u16x2 el = {(ushort)(se & 7u), (ushort)(se & 7u)}, eh = {(ushort)(se >> 3), (ushort)(se >> 3)};
                            const gq_u16x2 ol = {(ushort)(so & 7u), (ushort)(so & 7u)}, oh = {(ushort)(so >> 3), (ushort)(so >> 3)};
                            const uint2 qq = cur.q[c];
                            const uint lx = qq.x & 0x0F0F0F0Fu, ly = qq.y & 0x0F0F0F0Fu;
                            const uint hx = (qq.x >> 4) & 0x0F0F0F0Fu, hy = (qq.y >> 4) & 0x0F0F0F0Fu;
                            BA[c] = (gq_i4){(int)gq_mul4(lx, el), (int)gq_mul4(ly, el), (int)gq_mul4(hx, ol), (int)gq_mul4(hy, ol)};
                            BB[c] = (gq_i4){(int)gq_mul4(lx, eh), (int)gq_mul4(ly, eh), (int)gq_mul4(hx, oh), (int)gq_mul4(hy, oh)};
                        }
#pragma unroll
                        for (int p = 0; p < P; p++) {
                            const uchar* xp = xa + (size_t)(16 * p) * S + s * 256u;
                            gq_i4 DA0 = zero, DA1 = zero, DB0 = zero, DB1 = zero;
#pragma unroll
                            for (int c = 0; c < 4; c += 2) {
                                const uint2 a00 = *(const uint2*)(xp + 64 * c), a01 = *(const uint2*)(xp + 64 * c + 32);
                                const uint2 a10 = *(const uint2*)(xp + 64 * c + 64), a11 = *(const uint2*)(xp + 64 * c + 96);
                                const gq_i4 A0 = {(int)a00.x, (int)a00.y, (int)a01.x, (int)a01.y};
                                const gq_i4 A1 = {(int)a10.x, (int)a10.y, (int)a11.x, (int)a11.y};
                                DA0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A0, BA[c], DA0, 0, 0, 0);
                                DB0 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A0, BB[c], DB0, 0, 0, 0);
                                DA1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A1, BA[c + 1], DA1, 0, 0, 0);
                                DB1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(A1, BB[c + 1], DB1, 0, 0, 0);
                            }
                            const uchar* pq = lbq + ((size_t)s * BM + 16u * p + n) * 16u;
                            // (masked, not branched over: a branch here splits the unrolled code into basic blocks and costs registers)
                            const long km_ = kg == 0u ? -1l : 0l;
                            const long Alo = *(const long*)pq & km_, Ahi = *(const long*)(pq + 8) & km_;
                            const gq_i4 Dlo = __builtin_amdgcn_mfma_i32_16x16x32_i8(Alo, Bm, zero, 0, 0, 0);
                            const gq_i4 Dhi = __builtin_amdgcn_mfma_i32_16x16x32_i8(Ahi, Bm, zero, 0, 0, 0);
                            const float4 sx = *(const float4*)(lsx + s * BM + 16u * p + 4u * kg);
                            const float sxv[4] = {sx.x, sx.y, sx.z, sx.w};
#pragma unroll
                            for (int v = 0; v < 4; v++) {
                                const int isum = 8 * (DB0[v] + DB1[v]) + (DA0[v] + DA1[v]);
                                acc[q][p][v] += sxv[v] * (d * (float)isum - dmin * (float)(64 * Dhi[v] + Dlo[v]));
                            }
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    } else {
                    int sc[8];
                    long B[8];
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        sc[c] = (int)((sc_lo >> (8 * c)) & 0xFFu);
                        sc[4 + c] = (int)((sc_hi >> (8 * c)) & 0xFFu);
                        B[2 * c] = gq_pack(cur.q[c].x & 0x0F0F0F0Fu, cur.q[c].y & 0x0F0F0F0Fu);
                        B[2 * c + 1] = gq_pack((cur.q[c].x >> 4) & 0x0F0F0F0Fu, (cur.q[c].y >> 4) & 0x0F0F0F0Fu);
                    }
#pragma unroll
                    for (int p = 0; p < P; p++) {
                        int isum[4] = {0, 0, 0, 0};
                        const uchar* xp = xa + (size_t)(16 * p) * S + s * 256u;
#pragma unroll
                        for (int jj = 0; jj < 8; jj++) {
                            const long A = *(const long*)(xp + 32 * jj);
                            const gq_i4 D = __builtin_amdgcn_mfma_i32_16x16x32_i8(A, B[jj], zero, 0, 0, 0);
#pragma unroll
                            for (int v = 0; v < 4; v++) isum[v] += __mul24(sc[jj], D[v]);
                        }
                        // token n of this pass: its eight lo parts, then its eight hi parts (lanes kg = 0 only)
                        const uchar* pq = lbq + ((size_t)s * BM + 16u * p + n) * 16u;
                        // (masked, not branched over: a branch here splits the unrolled code into basic blocks and costs registers)
                        const long km_ = kg == 0u ? -1l : 0l;
                        const long Alo = *(const long*)pq & km_, Ahi = *(const long*)(pq + 8) & km_;
                        const gq_i4 Dlo = __builtin_amdgcn_mfma_i32_16x16x32_i8(Alo, Bm, zero, 0, 0, 0);
                        const gq_i4 Dhi = __builtin_amdgcn_mfma_i32_16x16x32_i8(Ahi, Bm, zero, 0, 0, 0);
                        const float4 sx = *(const float4*)(lsx + s * BM + 16u * p + 4u * kg);
                        acc[q][p][0] += sx.x * (d * (float)isum[0] - dmin * (float)(64 * Dhi[0] + Dlo[0]));
                        acc[q][p][1] += sx.y * (d * (float)isum[1] - dmin * (float)(64 * Dhi[1] + Dlo[1]));
                        acc[q][p][2] += sx.z * (d * (float)isum[2] - dmin * (float)(64 * Dhi[2] + Dlo[2]));
                        acc[q][p][3] += sx.w * (d * (float)isum[3] - dmin * (float)(64 * Dhi[3] + Dlo[3]));
                        // (keeps the passes apart: let loose, the scheduler hoists every pass's reads and
                        // products to the front and the kernel spills)
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    }
                    cur = nx;
                    // the tokens are read from LDS again for the next row tile: kept in registers across
                    // row tiles (which the compiler would do) they cost 96 registers and the kernel spills
                    if (RT > 1) asm volatile("" ::: "memory");
                }
            }
        }
        // K-slices of a row tile meet in LDS, added in slice order
        if (KW > 1u) {
#pragma unroll
            for (int q = 0; q < RT; q++)
#pragma unroll
                for (int p = 0; p < P; p++)
#pragma unroll
                    for (int v = 0; v < 4; v++) red[(((wave * RT + q) * P + p) * 4 + v) * 64u + lane] = acc[q][p][v];
            __syncthreads();
            if (kw == 0u) {
#pragma unroll
                for (int q = 0; q < RT; q++)
#pragma unroll
                    for (int p = 0; p < P; p++)
#pragma unroll
                        for (int v = 0; v < 4; v++) {
                            float t = acc[q][p][v];
                            for (uint k2 = 1; k2 < KW; k2++) t += red[((((wave + k2) * RT + q) * P + p) * 4 + v) * 64u + lane];
                            acc[q][p][v] = t;
                        }
            }
            __syncthreads();                                     // before the next group writes `red`
        }
        if (kw == 0u) {
#pragma unroll
            for (int q = 0; q < RT; q++) {
                const uint r_out = (tile0 + (uint)q * RW) * 16u + n;
#pragma unroll
                for (int p = 0; p < P; p++)
#pragma unroll
                    for (int v = 0; v < 4; v++) {
                        const uint t = t0 + 16u * p + 4u * kg + v;
                        if (t < M && r_out < N) {
                            float* o = y + (size_t)t * N + r_out;
                            *o = ACC ? *o + acc[q][p][v] : acc[q][p][v];
                        }
                    }
            }
        }
    }
}

// (Only RT = 1 is built.  With four row tiles per wave a staged chunk of tokens would serve 256 rows,
// which is what a batch of hundreds of tokens needs — at 64 rows per workgroup the re-staging of the
// tokens is the larger stream — but that instance needs more than 256 registers as compiled, spills and
// runs ten times slower.)
// (at least two waves per SIMD: with a register budget of 256 the matrix-core results are written
// to ordinary registers instead of the accumulation file, which saves a move per result)
extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 8)))
gemm_q8k_q4k_mf(const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N, uint M, uint ACC,
                uint RW, uint RT) {
    __shared__ __attribute__((aligned(16))) uchar lds_gq[GQ_LDS];
    const uint left = M - min(M, blockIdx.y * 64u);              // tokens of this workgroup's tile
    (void)RT;                                                    // only one row tile per wave is built
    if (left <= 16u) gemm_q8k_q4k_mf_body<1, 1>(xq, xs, w, y, K, N, M, ACC, RW, lds_gq);
    else if (left <= 32u) gemm_q8k_q4k_mf_body<2, 1>(xq, xs, w, y, K, N, M, ACC, RW, lds_gq);
    else gemm_q8k_q4k_mf_body<4, 1>(xq, xs, w, y, K, N, M, ACC, RW, lds_gq);
}

// What the two entries below stage once per workgroup: token rows 0 .. M - 1 (S bytes apart, eight
// loads in flight per thread), scales [sb][16] and split sums [sb][16][16] (zero from token M on).
__device__ __forceinline__ void gq_stage16(uchar* lds, float* lsx, uchar* lbq, const signed char* __restrict__ xq,
                                           const float* __restrict__ xs, uint K, uint S, uint M) {
    const uint nsb = K >> 8, per_row = K >> 4, total = M * per_row, nt = blockDim.x, tid = threadIdx.x;
    for (uint i0 = tid; i0 < total; i0 += 8u * nt) {
        uint4 v[8];
        uint dst[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const uint i = i0 + (uint)u * nt, t = i / per_row, o = (i - t * per_row) << 4;
            v[u] = make_uint4(0u, 0u, 0u, 0u);
            dst[u] = t * S + o;
            if (i < total) v[u] = *(const uint4*)(xq + (size_t)t * K + o);
        }
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (i0 + (uint)u * nt < total) *(uint4*)(lds + dst[u]) = v[u];
    }
    for (uint i = tid; i < nsb * 16u; i += nt) {
        const uint sb = i >> 4, t = i & 15u;
        lsx[i] = t < M ? xs[(size_t)t * nsb + sb] : 0.0f;
    }
    __syncthreads();
    // bsum of every (token, sub-block), split into int8 parts: 64 * hi + lo
    for (uint i = tid; i < nsb * 128u; i += nt) {
        const uint jj = i & 7u, t = (i >> 3) & 15u, s = i >> 7;
        int bs = 0;
        if (t < M) {
            const uint4* px = (const uint4*)(lds + (size_t)t * S + s * 256u + jj * 32u);
            const uint4 a = px[0], b = px[1];
            bs = dot4_i8(a.x, 0x01010101u, 0);
            bs = dot4_i8(a.y, 0x01010101u, bs); bs = dot4_i8(a.z, 0x01010101u, bs); bs = dot4_i8(a.w, 0x01010101u, bs);
            bs = dot4_i8(b.x, 0x01010101u, bs); bs = dot4_i8(b.y, 0x01010101u, bs);
            bs = dot4_i8(b.z, 0x01010101u, bs); bs = dot4_i8(b.w, 0x01010101u, bs);
        }
        uchar* o = lbq + ((size_t)s * 16u + t) * 16u;
        o[jj] = (uchar)(bs & 63);
        o[8u + jj] = (uchar)(bs >> 6);
    }
    __syncthreads();
}

// ---- up to 16 tokens, rows copied through LDS --------------------------------------------------
//   gemm_q8k_q4k_ml(xq, xs, w, y, K, N, M, ACC)   M <= 16, block 64 .. 512, w 16-byte aligned, rows within 4 GiB,
//                                                 16 (K + 32) + 5 K / 4 + 256 + 73728 <= 163840
// On a long matrix (an output head) and few tokens gemm_q8k_q4k_mf is bound by the address
// path of its loads (8-byte pieces of sixteen rows 144 K / 256 bytes apart: the unit that walks
// them is busy 85 % of the launch).  Here the memory system copies the rows instead: a wave owns
// 16-row tiles and a ring of four units in LDS (one unit = its 16 rows at one super-block,
// 2304 bytes, three global_load_lds_dwordx4 of nine lanes per row), walks its tiles as one stream
// of units with the copies three units ahead across tile borders, and never waits for another
// wave once the tokens are staged.  Rows land 144 bytes apart: 36 n mod 64 is a different multiple
// of four for each of the sixteen rows, so header and code reads spread evenly over the banks.
// The arithmetic per super-block is gemm_q8k_q4k_mf's; super-blocks are added in order (its
// RW = 4 form: the same bits).
#define GQL_UNIT 2304u
#define GQL_DEPTH 4u
#define GQL_LDS 163840u

extern "C" __global__ void __launch_bounds__(512)
gemm_q8k_q4k_ml(const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {
    __shared__ __attribute__((aligned(16))) uchar lds[GQL_LDS];
    const uint lds_addr = (uint)(size_t)(__attribute__((address_space(3))) uchar*)lds;
    const uint tid = threadIdx.x, lane = tid & 63u;
    const uint wave = (uint)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint nsb = K >> 8, S = K + 32u;
    const uint o_lsx = 16u * S, o_lbq = o_lsx + nsb * 64u, o_zero = o_lbq + nsb * 256u;
    const uint o_ring = o_zero + 256u + wave * (GQL_DEPTH * GQL_UNIT);
    float* lsx = (float*)(lds + o_lsx);            // [sb][16] token scales
    uchar* lbq = lds + o_lbq;                      // [sb][16][16]: lo_0..7, hi_0..7 of the bsums
    if (tid < 64u) ((uint*)(lds + o_zero))[tid] = 0u;   // what the A lanes of tokens past M read
    gq_stage16(lds, lsx, lbq, xq, xs, K, S, M);    // (its last barrier: every load so far is older than the copies)
    // wave ids interleave over the workgroups, so each CU gets its share of the waves with one tile more
    const uint tiles = (N + 15u) >> 4, stride = gridDim.x * (blockDim.x >> 6), first = wave * gridDim.x + blockIdx.x;
    const uint my_tiles = first < tiles ? (tiles - first + stride - 1u) / stride : 0u;
    const uint total = my_tiles * nsb;             // units this wave walks
    const uint row_bytes = nsb * Q4K_BYTES;
    // the copy stream: nine lanes per row, seven rows per copy (rows 14 and 15 in the third)
    const uint cq = lane / 9u, cpc = lane - cq * 9u;
    uint i_off[3], iu = 0u, i_sb = 0u, i_tile = first, i_slot = 0u;
    auto issue_next = [&]() {
        if (i_sb == 0u) {
#pragma unroll
            for (uint i = 0; i < 3u; i++) i_off[i] = min(i_tile * 16u + min(7u * i + cq, 15u), N - 1u) * row_bytes + cpc * 16u;
        }
        const uint dst = lds_addr + o_ring + i_slot * GQL_UNIT;
        if (lane < 63u) {
            lds_dma16(w, i_off[0] + i_sb * Q4K_BYTES, dst);
            lds_dma16(w, i_off[1] + i_sb * Q4K_BYTES, dst + 1008u);
        }
        if (lane < 18u) lds_dma16(w, i_off[2] + i_sb * Q4K_BYTES, dst + 2016u);
        iu++;
        i_slot = i_slot + 1u == GQL_DEPTH ? 0u : i_slot + 1u;
        if (++i_sb == nsb) {
            i_sb = 0u;
            i_tile += stride;
        }
    };
    for (uint k = 0; k + 1u < GQL_DEPTH; k++)
        if (iu < total) issue_next();
    const uint n = lane & 15u, kg = lane >> 4;
    const uchar* xa = n < M ? lds + (size_t)n * S + 8u * kg : lds + o_zero + 8u * kg;
    const uint xstep = n < M ? 256u : 0u;
    const uchar* rd = lds + o_ring + n * Q4K_BYTES;
    float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    uint c_sb = 0u, c_tile = first, c_slot = 0u;
    for (uint u = 0; u < total; u++) {
        if (iu < total) issue_next();              // unit u + 3, into the slot read during unit u - 1
        vm_wait(min(total - 1u - u, GQL_DEPTH - 1u) * 3u);
        const uchar* blk = rd + c_slot * GQL_UNIT;
        c_slot = c_slot + 1u == GQL_DEPTH ? 0u : c_slot + 1u;
        GqW cur;
        cur.hdr = *(const uint4*)blk;
#pragma unroll
        for (int c = 0; c < 4; c++) cur.q[c] = *(const uint2*)(blk + 16u + 32u * c + 8u * kg);
        gq_superblock(cur, xa + c_sb * xstep, lbq + ((size_t)c_sb * 16u + n) * 16u, lsx + c_sb * 16u, kg, acc);
        if (++c_sb == nsb) {
            const uint r_out = c_tile * 16u + n;
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const uint t = 4u * kg + v;
                if (t < M && r_out < N) {
                    float* o = y + (size_t)t * N + r_out;
                    *o = ACC ? *o + acc[v] : acc[v];
                }
                acc[v] = 0.0f;
            }
            c_sb = 0u;
            c_tile += stride;
        }
    }
}

// ---- up to 16 tokens on few rows: a tile's super-blocks split over the workgroup's waves --------
//   gemm_q8k_q4k_mk(xq, xs, w, y, K, N, M, ACC)   M <= 16, block 512, M (K + 32) + 5 K / 4 + 256 + 8192 <= 163840
// A projection of a few thousand rows has fewer 16-row tiles than the GPU has waves.  Here a
// workgroup owns a tile (tiles grid-stride): wave w takes super-blocks w, w + 8, ... against all the
// tokens, and the eight partial sums meet in LDS, added in wave order.  The whole of LDS belongs to
// the one workgroup of a CU, so the M tokens wait there whole (8 tokens of K = 14336); token rows
// past M are one shared block of zeros.
extern "C" __global__ void __launch_bounds__(512)
gemm_q8k_q4k_mk(const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) {
    __shared__ __attribute__((aligned(16))) uchar lds[GQL_LDS];
    const uint tid = threadIdx.x, lane = tid & 63u;
    const uint wave = (uint)__builtin_amdgcn_readfirstlane((int)(tid >> 6)), nw = blockDim.x >> 6;
    const uint nsb = K >> 8, S = K + 32u;
    const uint o_lsx = M * S, o_lbq = o_lsx + nsb * 64u, o_zero = o_lbq + nsb * 256u, o_red = o_zero + 256u;
    float* lsx = (float*)(lds + o_lsx);            // [sb][16] token scales
    uchar* lbq = lds + o_lbq;                      // [sb][16][16]: lo_0..7, hi_0..7 of the bsums
    float* red = (float*)(lds + o_red);            // [wave][4][64]
    if (tid < 64u) ((uint*)(lds + o_zero))[tid] = 0u;
    gq_stage16(lds, lsx, lbq, xq, xs, K, S, M);
    const uint n = lane & 15u, kg = lane >> 4;
    const uchar* xa = n < M ? lds + (size_t)n * S + 8u * kg : lds + o_zero + 8u * kg;
    const uint xstep = n < M ? 256u : 0u;
    const uint tiles = (N + 15u) >> 4;
    for (uint tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        const uint row = min(tile * 16u + n, N - 1u);
        const uchar* wr = w + (size_t)row * nsb * Q4K_BYTES;
        float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        // (one super-block ahead; two ahead, and loads skipped rather than clamped past the slice, measured the same)
        GqW cur = gq_load(wr + (size_t)min(wave, nsb - 1u) * Q4K_BYTES, kg);
        for (uint sb = wave; sb < nsb; sb += nw) {
            const GqW nx = gq_load(wr + (size_t)min(sb + nw, nsb - 1u) * Q4K_BYTES, kg);
            gq_superblock(cur, xa + sb * xstep, lbq + ((size_t)sb * 16u + n) * 16u, lsx + sb * 16u, kg, acc);
            cur = nx;
        }
#pragma unroll
        for (int v = 0; v < 4; v++) red[(wave * 4u + (uint)v) * 64u + lane] = acc[v];
        __syncthreads();
        if (tid < 256u) {
            const uint l = tid & 63u, v = tid >> 6;
            float sum = red[v * 64u + l];
            for (uint w8 = 1; w8 < nw; w8++) sum += red[(w8 * 4u + v) * 64u + l];
            const uint t = 4u * (l >> 4) + v, r_out = tile * 16u + (l & 15u);
            if (t < M && r_out < N) {
                float* o = y + (size_t)t * N + r_out;
                *o = ACC ? *o + sum : sum;
            }
        }
        __syncthreads();                           // before the next tile's partial sums
    }
}

// ---- prefill-sized batches: 128 tokens x 128 rows per workgroup, tokens copied into LDS by the memory system ----
//   q8k_token_sides(xq, xs, xst, sums, K, M, MP)      grid [K / 256, ceil(MP / 256), 1], block 256
//       xst [K/256][MP] f32: the token scales, super-block major;  sums [K/256][MP][8] f32: scale x every 32-position
//       sum of a token's activations, in the order 0 4 1 5 2 6 3 7; rows M .. MP - 1 are zeros.
//   gemm_q8k_q4k_xt(xq, xst, sums, w, y, K, N, M, ACC, MP)    grid [ceil(N / 128), MP / 128, 1], block 512;  MP = M rounded up to 128
//   gemm_q8k_q4k_xt64(the same)                                grid [ceil(N / 64), MP / 128, 1]
//
// gemm_q8k_q4k_mf stages its tokens through registers, one chunk of K at a time, with nothing else going on: from
// a hundred tokens up that staging, not the arithmetic, is what the launch waits for.  Here a workgroup owns
// 128 tokens x 128 rows and walks K one super-block per step; the step's tokens (32 KB), their scales and split
// sums travel global -> LDS by global_load_lds_dwordx4 into the stage the previous step is not reading, and are
// awaited with one s_waitcnt + barrier per step.  A token row is 256 bytes; its 16-byte piece j sits in slot
// j ^ (token % 16), applied on the global side of the copy, so that the sixteen tokens of a pass read a given piece
// from sixteen different bank groups.  A wave owns one 16-row tile and the eight passes of 16 tokens (the _xt64 entry:
// 64 rows per workgroup, two waves per tile with four passes each, for matrices with few rows): the tile's
// weights, scales folded into two int8 planes (see gemm_q8k_q4k_mf), are built once per step, and every 16 bytes of
// activations read from LDS feed two v_mfma_i32_16x16x64_i8 (the two planes).  The weights of the next step
// are ordinary loads into registers, issued a step ahead.  Per (token, row, super-block) the sum takes
//     - sum_j (xs bsum_j) (dmin m_j)     two v_mfma_f32_16x16x4_f32 onto the running sums, factors rounded to f32 once
//     + xs (d isum)                      isum exact in int32
// super-blocks in order: gemm_q8k_q4k_mf's terms with the min part associated per run instead of per super-block
// (a few ulp of the result apart; four vector instructions per result and super-block instead of seven).
#define GXT_TOK 128u
#define GXT_ROWS 128u
#define GXT_STAGE (GXT_TOK * 256u + GXT_TOK * 32u + GXT_TOK * 4u)     // tokens | scaled sums | scales = 37376 bytes

extern "C" __global__ void __launch_bounds__(256)
q8k_token_sides(const signed char* __restrict__ xq, const float* __restrict__ xs, float* __restrict__ xst,
                float* __restrict__ sums, uint K, uint M, uint MP) {
    const uint nsb = K >> 8, sb = blockIdx.x, t = blockIdx.y * 256u + threadIdx.x;
    if (t >= MP) return;
    float f[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
    float sc = 0.0f;
    if (t < M) {
        sc = xs[(size_t)t * nsb + sb];
        const uint4* px = (const uint4*)(xq + (size_t)t * K + (size_t)sb * 256u);
#pragma unroll
        for (int jj = 0; jj < 8; jj++) {
            const uint4 a = px[2 * jj], b = px[2 * jj + 1];
            int bs = dot4_i8(a.x, 0x01010101u, 0);
            bs = dot4_i8(a.y, 0x01010101u, bs); bs = dot4_i8(a.z, 0x01010101u, bs); bs = dot4_i8(a.w, 0x01010101u, bs);
            bs = dot4_i8(b.x, 0x01010101u, bs); bs = dot4_i8(b.y, 0x01010101u, bs);
            bs = dot4_i8(b.z, 0x01010101u, bs); bs = dot4_i8(b.w, 0x01010101u, bs);
            f[2 * (jj & 3) + (jj >> 2)] = __fmul_rn(sc, (float)bs);
        }
    }
    xst[(size_t)sb * MP + t] = sc;
    float4* o = (float4*)(sums + ((size_t)sb * MP + t) * 8u);
    o[0] = make_float4(f[0], f[1], f[2], f[3]);
    o[1] = make_float4(f[4], f[5], f[6], f[7]);
}

// The activation quantizer and q8k_token_sides in one launch, for callers that hand over f32 or bf16 tokens:
//   quantize_q8k{,_bf16}_sides(x, q, scales, xst, sums, K, M, MP)    grid [K / 256 * MP / 4, 1, 1], block 256
// One wave per 256-segment, segments numbered token-major (segment s = token s / (K / 256), super-block s % (K / 256)),
// four values per lane: the segment is quantized exactly as quantize_q8k does (amax / 127, 1 for a zero segment, round
// half away, clamp), and its scale and scaled 32-position sums go to the transposed side arrays as well; the segments of
// rows M .. MP - 1 write zeros there and nothing else.  No barrier and no LDS: the maximum and the sums travel by DPP.
template <bool BF16>
__device__ __forceinline__ void quantize_q8k_sides_body(const void* __restrict__ xv, signed char* __restrict__ q,
                                                        float* __restrict__ scales, float* __restrict__ xst,
                                                        float* __restrict__ sums, uint K, uint M, uint MP) {
    const uint nsb = K >> 8, lane = threadIdx.x & 63u;
    const uint seg = blockIdx.x * 4u + (threadIdx.x >> 6);
    const uint m = seg / nsb, sb = seg - m * nsb;
    if (m >= MP) return;
    if (m >= M) {
        if (lane == 0) xst[(size_t)sb * MP + m] = 0.0f;
        if (lane < 8u) sums[((size_t)sb * MP + m) * 8u + lane] = 0.0f;
        return;
    }
    const size_t i = (size_t)seg * 256u + lane * 4u;
    float v[4];
    if (BF16) {
        const uint2 b = *(const uint2*)((const ushort*)xv + i);
        v[0] = __uint_as_float(b.x << 16);
        v[1] = __uint_as_float(b.x & 0xFFFF0000u);
        v[2] = __uint_as_float(b.y << 16);
        v[3] = __uint_as_float(b.y & 0xFFFF0000u);
    } else {
        const float4 f = *(const float4*)((const float*)xv + i);
        v[0] = f.x, v[1] = f.y, v[2] = f.z, v[3] = f.w;
    }
    const float mx = wave_max(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))));
    const float scale = mx > 0.0f ? __fdiv_rn(mx, 127.0f) : 1.0f;
    const float inv = __fdiv_rn(1.0f, scale);
    int s32 = 0;
    uint pk = 0;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int r = (int)sat127(roundf(__fmul_rn(v[e], inv)));
        s32 += r;
        pk |= ((uint)r & 0xFFu) << (8 * e);
    }
    *(uint*)(q + i) = pk;
    // eight lanes hold one run of 32 positions
    s32 += dpp_i32<OJK_DPP_QUAD_XOR1>(s32);
    s32 += dpp_i32<OJK_DPP_QUAD_XOR2>(s32);
    s32 += dpp_i32<OJK_DPP_ROW_HALF_MIRROR>(s32);
    // lane 8 j holds the sum of run j, which goes to position 2 (j % 4) + j / 4
    if ((lane & 7u) == 0) sums[((size_t)sb * MP + m) * 8u + ((lane >> 2) & 6u) + (lane >> 5)] = __fmul_rn(scale, (float)s32);
    if (lane == 0) {
        scales[seg] = scale;
        xst[(size_t)sb * MP + m] = scale;
    }
}
extern "C" __global__ void __launch_bounds__(256)
quantize_q8k_sides(const float* x, signed char* q, float* scales, float* xst, float* sums, uint K, uint M, uint MP) {
    quantize_q8k_sides_body<false>(x, q, scales, xst, sums, K, M, MP);
}
extern "C" __global__ void __launch_bounds__(256)
quantize_q8k_bf16_sides(const ushort* x, signed char* q, float* scales, float* xst, float* sums, uint K, uint M, uint MP) {
    quantize_q8k_sides_body<true>(x, q, scales, xst, sums, K, M, MP);
}

__device__ __forceinline__ void gxt_copy16(const void* base, uint voff, uint lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(base), "s"(lds_addr) : "memory");
}

// the two planes of one 16-row tile's super-block: BA = (sc & 7) * code, BB = (sc >> 3) * code, a chunk per register quad;
// and the row's side of the min term for the f32 matrix unit: n0 = -dmin * m[kg], n1 = -dmin * m[kg + 4] (sh = 8 kg)
__device__ __forceinline__ void gxt_planes(const GqW& w, gq_i4 (&BA)[4], gq_i4 (&BB)[4], float& n0, float& n1, float& d, uint sh) {
    d = f16_bits_to_f32(w.hdr.x & 0xFFFFu);
    const float ndmin = -f16_bits_to_f32(w.hdr.x >> 16);
    const uint sc_lo = w.hdr.y & 0x3F3F3F3Fu, mn_lo = w.hdr.z & 0x3F3F3F3Fu;
    const uint sc_hi = (w.hdr.w & 0x0F0F0F0Fu) | ((w.hdr.y >> 2) & 0x30303030u);
    const uint mn_hi = ((w.hdr.w >> 4) & 0x0F0F0F0Fu) | ((w.hdr.z >> 2) & 0x30303030u);
    n0 = __fmul_rn(ndmin, (float)((mn_lo >> sh) & 0xFFu));
    n1 = __fmul_rn(ndmin, (float)((mn_hi >> sh) & 0xFFu));
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const uint se = 2 * c < 4 ? (sc_lo >> (16 * c)) & 0xFFu : (sc_hi >> (16 * (c - 2))) & 0xFFu;
        const uint so = 2 * c < 4 ? (sc_lo >> (16 * c + 8)) & 0xFFu : (sc_hi >> (16 * (c - 2) + 8)) & 0xFFu;
        const gq_u16x2 el = {(ushort)(se & 7u), (ushort)(se & 7u)}, eh = {(ushort)(se >> 3), (ushort)(se >> 3)};
        const gq_u16x2 ol = {(ushort)(so & 7u), (ushort)(so & 7u)}, oh = {(ushort)(so >> 3), (ushort)(so >> 3)};
        const uint2 qq = w.q[c];
        const uint lx = qq.x & 0x0F0F0F0Fu, ly = qq.y & 0x0F0F0F0Fu;
        const uint hx = (qq.x >> 4) & 0x0F0F0F0Fu, hy = (qq.y >> 4) & 0x0F0F0F0Fu;
        BA[c] = (gq_i4){(int)gq_mul4(lx, el), (int)gq_mul4(ly, el), (int)gq_mul4(hx, ol), (int)gq_mul4(hy, ol)};
        BB[c] = (gq_i4){(int)gq_mul4(lx, eh), (int)gq_mul4(ly, eh), (int)gq_mul4(hx, oh), (int)gq_mul4(hy, oh)};
    }
}

// TH = 1: eight row tiles (128 rows) per workgroup, a wave takes one of them against all eight passes of 16 tokens;
// TH = 2: four row tiles (64 rows), two waves per tile with four passes each — for matrices with too few rows to give
// every CU a 128-row tile.
// SPLIT: the workgroup takes slice blockIdx.z of the super-blocks; the slices' partial tiles meet in `part`, one counter
// per tile in `cnt` (zero before the first launch, every launch leaves zeros): the slice that finds all the others
// counted adds them in slice order — its own read back too, so the sum does not depend on who came last — and owns y.
template <int TH, bool SPLIT = false>
__device__ __forceinline__ void gemm_q8k_q4k_xt_body(const signed char* __restrict__ xq, const float* __restrict__ xst,
                                                     const float* __restrict__ sums, const uchar* __restrict__ w,
                                                     float* __restrict__ y, uint K, uint N, uint M, uint ACC, uint MP, uchar* lds,
                                                     float* __restrict__ part = nullptr, uint* __restrict__ cnt = nullptr,
                                                     uint nsplit = 1u) {
    constexpr int P = 8 / TH;
    constexpr uint RT = 8u / TH;                                    // row tiles per workgroup
    const uint tid = threadIdx.x, lane = tid & 63u;
    const uint wave = (uint)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint rt = wave % RT, th = wave / RT;                     // the wave's 16 rows and its 16 P tokens
    const uint nsb = K >> 8, n = lane & 15u, kg = lane >> 4;
    const uint t0 = blockIdx.y * GXT_TOK, r0 = blockIdx.x * (16u * RT) + rt * 16u;
    const uint lds0 = (uint)(size_t)(__attribute__((address_space(3))) uchar*)lds;
    const gq_i4 zero = {0, 0, 0, 0};

    // copies of one step: 32 of 1 KB for the tokens (wave w takes tokens 16 w .. 16 w + 15, four per copy: lane ->
    // token lane / 16 of the four, slot lane % 16, which holds the token's piece slot ^ (token % 16)), four for the
    // scaled sums (128 tokens x 32 bytes, contiguous in `sums`), one of 512 bytes for the scales.
    const uint lane16 = lane * 16u;
    const uint x_lds = lds0 + wave * 4096u;                        // + stage * GXT_STAGE + i * 1024
    auto copies = [&](uint sb, uint stage) {
        const uchar* xb = (const uchar*)xq + (size_t)sb * 256u;
        // (the four source offsets are formed again at every step — a dozen instructions — rather than kept in
        // registers across the loop, which this kernel does not have: the lane id is made opaque to stop the hoisting)
        uint lo = lane;
        asm volatile("" : "+v"(lo));
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint tk = wave * 16u + (uint)i * 4u + (lo >> 4);
            const uint tg = min(t0 + tk, M - 1u);                  // tokens past M: any row (their sides are zeros)
            gxt_copy16(xb, tg * K + (((lo & 15u) ^ (tk & 15u)) << 4), x_lds + stage * GXT_STAGE + (uint)i * 1024u);
        }
        if (wave < 4u) gxt_copy16((const uchar*)sums + ((size_t)sb * MP + t0) * 32u + wave * 1024u, lane16,
                                  lds0 + stage * GXT_STAGE + GXT_TOK * 256u + wave * 1024u);
        else if (wave == 4u) {
            if (lane < 32u) gxt_copy16(xst + (size_t)sb * MP + t0, lane16, lds0 + stage * GXT_STAGE + GXT_TOK * 288u);
        }
    };
    // this lane's row (clamped past N; a 32-bit byte offset from a uniform base: the tensor stays below 4 GiB)
    const uint wrow = min(r0 + n, N - 1u) * nsb * Q4K_BYTES;

    gq_f4 acc[P];
#pragma unroll
    for (int p = 0; p < P; p++) acc[p] = (gq_f4){0.0f, 0.0f, 0.0f, 0.0f};

    // byte offsets of the lane's pieces within a token row, per chunk: pieces 4 c + kg / 2 (first sub-block) and
    // 4 c + 2 + kg / 2 (second), slot = piece ^ (token % 16), half kg % 2
    const uint tok_lds = (th * (16u * P) + n) * 256u + 8u * (kg & 1u);
    // (the second piece's slot differs from the first's in bit 1 only: its byte offset is the first's ^ 32)
    uint o0[4];
#pragma unroll
    for (int c = 0; c < 4; c++) o0[c] = tok_lds + (((4u * (uint)c + (kg >> 1)) ^ n) << 4);
    // the lane's two scaled sums of its token (runs kg and kg + 4 sit side by side), and the scales of the four tokens
    // whose results it holds
    const uint side_lds = GXT_TOK * 256u + (th * (16u * P) + n) * 32u + 8u * kg, sc_lds = GXT_TOK * 288u + (th * (16u * P) + 4u * kg) * 4u;
    const uint sh = 8u * kg;

    // the super-blocks of this workgroup: all of them, or slice blockIdx.z of ceil(nsb / nsplit) each
    const uint per = SPLIT ? (nsb + nsplit - 1u) / nsplit : nsb;
    const uint sb0 = SPLIT ? blockIdx.z * per : 0u, sb1 = SPLIT ? min(nsb, sb0 + per) : nsb;

    GqW cur = gq_load((w + (size_t)sb0 * Q4K_BYTES) + wrow, kg);
    copies(sb0, 0u);
    for (uint sb = sb0; sb < sb1; sb++) {
        const uint stage = (sb - sb0) & 1u;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();                                            // stage `stage` complete; the other one is free
        if (sb + 1u < sb1) copies(sb + 1u, stage ^ 1u);
        const uint sbn = min(sb + 1u, sb1 - 1u);
        const uchar* st = lds + stage * GXT_STAGE;
        gq_i4 BA[4], BB[4];
        float n0, n1, d;
        gxt_planes(cur, BA, BB, n0, n1, d, sh);
        __builtin_amdgcn_sched_barrier(0);
        // the next step's weights take over the registers of this step's raw bytes, which the planes have replaced
        cur = gq_load((w + (size_t)sbn * Q4K_BYTES) + wrow, kg);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int p = 0; p < P; p++) {
            // (one accumulation chain per plane: the two chains alternate, which is distance enough between dependent
            // MFMAs here, and saves the registers and the additions of split chains)
            // the min term goes straight onto the sums through the f32 matrix unit: - sum_j (xs bsum_j) (dmin m_j)
            const float2 am = *(const float2*)(st + side_lds + 512u * (uint)p);
            acc[p] = __builtin_amdgcn_mfma_f32_16x16x4f32(am.x, n0, acc[p], 0, 0, 0);
            acc[p] = __builtin_amdgcn_mfma_f32_16x16x4f32(am.y, n1, acc[p], 0, 0, 0);
            gq_i4 DA = zero, DB = zero;
#pragma unroll
            for (int c = 0; c < 4; c++) {
                const uint2 a0 = *(const uint2*)(st + o0[c] + 4096u * (uint)p), a1 = *(const uint2*)(st + (o0[c] ^ 32u) + 4096u * (uint)p);
                const gq_i4 A = {(int)a0.x, (int)a0.y, (int)a1.x, (int)a1.y};
                DA = __builtin_amdgcn_mfma_i32_16x16x64_i8(A, BA[c], DA, 0, 0, 0);
                DB = __builtin_amdgcn_mfma_i32_16x16x64_i8(A, BB[c], DB, 0, 0, 0);
            }
            const float4 sx = *(const float4*)(st + sc_lds + 64u * (uint)p);
            const float sxv[4] = {sx.x, sx.y, sx.z, sx.w};
#pragma unroll
            for (int v = 0; v < 4; v++) acc[p][v] += sxv[v] * (d * (float)(8 * DB[v] + DA[v]));
            // (keeps the passes apart: let loose, the scheduler hoists every pass's reads to the front)
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    if (SPLIT) {
        // The partial tile goes out as the registers hold it ([pair][thread]: 512 contiguous bytes per wave and store),
        // written through and read from behind the L2 (system-scope accesses): a tile's slices run on different XCDs,
        // whose L2s do not see each other's lines.  The stores are awaited by instruction before the slice is counted.
        typedef unsigned long long u64;
        const uint ns_eff = (nsb + per - 1u) / per;
        const uint tile = blockIdx.y * gridDim.x + blockIdx.x;
        const uint te = threadIdx.x;
        u64* const mine = (u64*)part + ((size_t)tile * ns_eff + blockIdx.z) * (uint)(P * 2) * 512u + te;
#pragma unroll
        for (int p = 0; p < P; p++)
#pragma unroll
            for (int h = 0; h < 2; h++)
                __hip_atomic_store(mine + (size_t)(p * 2 + h) * 512u,
                                   (u64)__float_as_uint(acc[p][2 * h]) | ((u64)__float_as_uint(acc[p][2 * h + 1]) << 32),
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        if (te == 0u) *(volatile uint*)lds = atomicAdd(cnt + tile, 1u);
        __syncthreads();
        if ((uint)__builtin_amdgcn_readfirstlane((int)*(volatile uint*)lds) != ns_eff - 1u) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        // (four slices' loads in flight before the first is added: a trip to memory per four slices, not one per load;
        // past the last slice the loads repeat it and are dropped)
        const u64* const all = (const u64*)part + (size_t)tile * ns_eff * (uint)(P * 2) * 512u + te;
        for (uint s0 = 0; s0 < ns_eff; s0 += 4u) {
            u64 v[4][P * 2];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const uint sl = min(s0 + (uint)q, ns_eff - 1u);
#pragma unroll
                for (int i = 0; i < P * 2; i++)
                    v[q][i] = __hip_atomic_load(all + ((size_t)sl * (uint)(P * 2) + (uint)i) * 512u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
#pragma unroll
            for (int q = 0; q < 4; q++) {
                if (s0 + (uint)q < ns_eff) {
#pragma unroll
                    for (int i = 0; i < P * 2; i++) {
                        const float a = __uint_as_float((uint)v[q][i]), b = __uint_as_float((uint)(v[q][i] >> 32));
                        const bool first = s0 + (uint)q == 0u;
                        acc[i / 2][2 * (i % 2)] = first ? a : acc[i / 2][2 * (i % 2)] + a;
                        acc[i / 2][2 * (i % 2) + 1] = first ? b : acc[i / 2][2 * (i % 2) + 1] + b;
                    }
                }
            }
        }
        if (te == 0u) cnt[tile] = 0u;                               // ready for the next launch
    }
    // (the lane id asked of the hardware again, so that nothing of it has to live through the loop)
    const uint le = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    const uint r = blockIdx.x * (16u * RT) + rt * 16u + (le & 15u);
#pragma unroll
    for (int p = 0; p < P; p++)
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const uint t = t0 + th * (16u * P) + 16u * (uint)p + 4u * (le >> 4) + (uint)v;
            if (t < M && r < N) {
                float* o = y + (size_t)t * N + r;
                *o = ACC ? *o + acc[p][v] : acc[p][v];
            }
        }
}

extern "C" __global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4)))
gemm_q8k_q4k_xt(const signed char* xq, const float* xst, const float* sums, const uchar* w, float* y, uint K, uint N, uint M,
                uint ACC, uint MP) {
    __shared__ __attribute__((aligned(1024))) uchar lds_xt[2 * GXT_STAGE];
    gemm_q8k_q4k_xt_body<1>(xq, xst, sums, w, y, K, N, M, ACC, MP, lds_xt);
}
extern "C" __global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4)))
gemm_q8k_q4k_xt64(const signed char* xq, const float* xst, const float* sums, const uchar* w, float* y, uint K, uint N, uint M,
                  uint ACC, uint MP) {
    __shared__ __attribute__((aligned(1024))) uchar lds_xt[2 * GXT_STAGE];
    gemm_q8k_q4k_xt_body<2>(xq, xst, sums, w, y, K, N, M, ACC, MP, lds_xt);
}
// the 64-row tile over K slices, for matrices whose 64-row tiles alone leave most CUs idle:
//   gemm_q8k_q4k_xt64_sr(xq, xst, sums, w, y, part, cnt, K, N, M, ACC, MP, NSPLIT)
//   grid [ceil(N / 64), MP / 128, slices]; slices = ceil(nsb / ceil(nsb / NSPLIT)); part: tiles x slices x 32 KB
extern "C" __global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4)))
gemm_q8k_q4k_xt64_sr(const signed char* xq, const float* xst, const float* sums, const uchar* w, float* y, float* part, uint* cnt,
                     uint K, uint N, uint M, uint ACC, uint MP, uint NSPLIT) {
    __shared__ __attribute__((aligned(1024))) uchar lds_xt[2 * GXT_STAGE];
    gemm_q8k_q4k_xt_body<2, true>(xq, xst, sums, w, y, K, N, M, ACC, MP, lds_xt, part, cnt, NSPLIT);
}

// ---- Q6_K and Q5_K rows against batches of tokens: one matrix instruction per scale group ---------------------------
//   gemm_q8k_{q6k,q5k}_gs(xq, xs, w, y, K, N, M, ACC)                      block 256, grid [ceil(N / 128), ceil(M / 64), 1]
//   gemm_q8k_{q6k,q5k}_gs_sr(xq, xs, w, y, part, cnt, K, N, M, ACC, NSPLIT)       grid [.., .., slices]
// The CPU path's arithmetic (dot_q6k / dot_q5k over quant_q8k activations, crates/ojas-cpu/src/cpu_math.rs:638-722) for
// batches from a handful of tokens to prefill sizes.  A Q6_K scale covers 16 weights and is a full int8, so it cannot be
// folded into int8 codes the way the Q4_K tile above folds its 6-bit scales; instead v_mfma_i32_32x32x16_i8, whose 16
// positions are exactly one scale group, gives the group's integer dots for 32 tokens x 32 rows, and the scale enters
// with one v_mad_i32_i24 per D register (the row is lane-constant in D).  Q5_K: one v_mfma_i32_32x32x32_i8 per 32-weight
// sub-block (codes 0..31 are one int8 plane), the 6-bit scale likewise, and sum_j m_j bsum_j from two more
// instructions per super-block over the sub-block sums split as 64 hi + lo (the workgroup splits them while it stages
// the tokens).
// A workgroup owns 128 rows x 64 tokens: wave w takes rows 32 w .. against both blocks of 32 tokens (only the first where
// the last token tile holds no more).  B (weights): lane (n, kg) = (lane % 32, lane / 32) builds the codes of
// positions 8 kg .. 8 kg + 7 of every group of row n from the raw bytes it loads itself, one super-block ahead — no two
// waves of a workgroup build the same codes.  A (tokens): a super-block's 64 x 256 int8 wait in LDS, rows 264 bytes
// apart (32 tokens' 8-byte reads then cover all banks), two stages, one barrier per super-block.  Integer sums are
// exact; per super-block acc += sx * d * (float) isum, super-blocks in order.
// `_sr`: K slices whose partial tiles meet in `part` (tiles x slices x 32 KB), added in slice order by the last to arrive.
#include "ojk_q6k_mfma.h"

typedef int gs_i16 __attribute__((ext_vector_type(16)));
#define GS_STRIDE 264u
#define GS_SX (64u * GS_STRIDE)         // the stage's 64 token scales
#define GS_BS (GS_SX + 256u)            // Q5_K: the split sub-block sums, 16 bytes per token (lo_0..7, hi_0..7)
#define GS_STAGE (GS_BS + 1024u)

// A running integer sum, pinned after every group: integer additions may be reassociated, and left to itself the
// compiler turns sixteen groups' multiply-adds into one tree at the end of the super-block, every group's sixteen result
// registers alive until then (hundreds of spills).
__device__ __forceinline__ int gs_pin(int v) {
    asm("" : "+v"(v));
    return v;
}

struct GsQ6K {
    static constexpr uint BYTES = Q6K_BYTES;
    static constexpr bool BSUMS = false;
    struct Raw {
        u32x2_a2 la[2][2], lb[2][2], qh[2][2];   // [half][group of the quarter]: ql[16 h + 8 kg ..], ql[32 + ..], qh[..]
        u32x4_a2 sc;
        uint d16;
    };
    static __device__ __forceinline__ Raw load(const uchar* blk, uint kg) {
        Raw r;
        const uint sh = ((uint)(size_t)blk & 2u) << 3;
        const uchar* b4 = blk - ((size_t)blk & 2u);
#pragma unroll
        for (int hf = 0; hf < 2; hf++)
#pragma unroll
            for (int h = 0; h < 2; h++) {
                r.la[hf][h] = q6k_ld8(b4 + 64u * hf + 16u * h + 8u * kg, sh);
                r.lb[hf][h] = q6k_ld8(b4 + 64u * hf + 32u + 16u * h + 8u * kg, sh);
                r.qh[hf][h] = q6k_ld8(b4 + 128u + 32u * hf + 16u * h + 8u * kg, sh);
            }
        const uint* ps = (const uint*)(b4 + 192u);
        const uint s0 = ps[0], s1 = ps[1], s2 = ps[2], s3 = ps[3], s4 = ps[4];
        r.sc.x = __builtin_amdgcn_alignbit(s1, s0, sh);
        r.sc.y = __builtin_amdgcn_alignbit(s2, s1, sh);
        r.sc.z = __builtin_amdgcn_alignbit(s3, s2, sh);
        r.sc.w = __builtin_amdgcn_alignbit(s4, s3, sh);
        r.d16 = (s4 >> sh) & 0xFFFFu;
        return r;
    }
    // st: the stage; tok0: the wave's first token in it
    template <int NB>   // NB: how many of the wave's two 32-token blocks hold tokens
    static __device__ __forceinline__ void superblock(const Raw& r, const uchar* st, uint tok0, uint fr, uint kg,
                                                      float (&acc)[2][16]) {
        const uchar* xa = st + (tok0 + fr) * GS_STRIDE + 8u * kg;            // the lane's token row of block 0, its 8 positions
        const float* sx = (const float*)(st + GS_SX) + tok0 + 4u * kg;       // scales of its D registers' tokens: + 32 i + 8 (v / 4) + v % 4
        int isum[NB][16];
#pragma unroll
        for (int i = 0; i < NB; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) isum[i][v] = 0;
        const gs_i16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        // group g = 8 hf + 2 q + h: quarter q of half hf, its positions 16 h .. 16 h + 15; scale byte g
        auto codes = [&](int g) -> long {
            const int hf = g >> 3, q = (g >> 1) & 3, h = g & 1;
            const u32x2_a2 ql = (q & 1) ? r.lb[hf][h] : r.la[hf][h];
            return q6k_signed8(ql.x, ql.y, r.qh[hf][h].x, r.qh[hf][h].y, q);
        };
        auto tokens = [&](int g, int i) -> long {
            return *(const long*)(xa + (uint)i * 32u * GS_STRIDE + 16u * (uint)g);
        };
        // the next group's operands are fetched and built under this group's matrix instructions, ahead of its multiply-adds
        long B = codes(0), A0 = tokens(0, 0), A1 = NB == 2 ? tokens(0, 1) : 0;
#pragma unroll
        for (int g = 0; g < 16; g++) {
            const uint sw = g < 4 ? r.sc.x : g < 8 ? r.sc.y : g < 12 ? r.sc.z : r.sc.w;
            const int s = (int)(signed char)(sw >> (8 * (g & 3)));
            const gs_i16 D0 = __builtin_amdgcn_mfma_i32_32x32x16_i8(A0, B, zero, 0, 0, 0);
            gs_i16 D1 = zero;
            if (NB == 2) D1 = __builtin_amdgcn_mfma_i32_32x32x16_i8(A1, B, zero, 0, 0, 0);
            if (g < 15) {
                A0 = tokens(g + 1, 0);
                if (NB == 2) A1 = tokens(g + 1, 1);
                B = codes(g + 1);
            }
#pragma unroll
            for (int v = 0; v < 16; v++) isum[0][v] = gs_pin(isum[0][v] + __mul24(s, D0[v]));
            if (NB == 2) {
#pragma unroll
                for (int v = 0; v < 16; v++) isum[NB - 1][v] = gs_pin(isum[NB - 1][v] + __mul24(s, D1[v]));
            }
            // (keeps the groups apart: let loose, the scheduler issues every group's matrix instructions first and
            // spills their results)
            __builtin_amdgcn_sched_barrier(0);
        }
        const float d = f16_bits_to_f32(r.d16);
#pragma unroll
        for (int i = 0; i < NB; i++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                // (spelled out: left to contract `acc += sx * d * isum` as it likes, the compiler fuses the last product
                // into the addition for one token block and not for the other, and a token's bits depend on its block)
                const float4 x4 = *(const float4*)(sx + 32 * i + 8 * g);
                acc[i][4 * g] = __fmaf_rn(__fmul_rn(x4.x, d), (float)isum[i][4 * g], acc[i][4 * g]);
                acc[i][4 * g + 1] = __fmaf_rn(__fmul_rn(x4.y, d), (float)isum[i][4 * g + 1], acc[i][4 * g + 1]);
                acc[i][4 * g + 2] = __fmaf_rn(__fmul_rn(x4.z, d), (float)isum[i][4 * g + 2], acc[i][4 * g + 2]);
                acc[i][4 * g + 3] = __fmaf_rn(__fmul_rn(x4.w, d), (float)isum[i][4 * g + 3], acc[i][4 * g + 3]);
            }
    }
};

struct GsQ5K {
    static constexpr uint BYTES = Q5K_BYTES;
    static constexpr bool BSUMS = true;
    struct Raw {
        uint4 hdr;          // d, dmin, the 12 scale bytes
        uint2 qh[2];        // fifth bits of positions 16 h + 8 kg .. + 7 (bit j: sub-block j)
        uint2 qs[4][2];     // [chunk][h]: nibbles of the same positions (low: sub-block 2 c, high: 2 c + 1)
    };
    static __device__ __forceinline__ Raw load(const uchar* blk, uint kg) {
        Raw r;
        r.hdr = *(const uint4*)blk;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            r.qh[h] = *(const uint2*)(blk + 16u + 16u * h + 8u * kg);
#pragma unroll
            for (int c = 0; c < 4; c++) r.qs[c][h] = *(const uint2*)(blk + 48u + 32u * c + 16u * h + 8u * kg);
        }
        return r;
    }
    template <int NB>   // NB: how many of the wave's two 32-token blocks hold tokens
    static __device__ __forceinline__ void superblock(const Raw& r, const uchar* st, uint tok0, uint fr, uint kg,
                                                      float (&acc)[2][16]) {
        const uchar* xa = st + (tok0 + fr) * GS_STRIDE + 8u * kg;            // the lane's token row of block 0, its 8 positions
        const float* sx = (const float*)(st + GS_SX) + tok0 + 4u * kg;       // scales of its D registers' tokens: + 32 i + 8 (v / 4) + v % 4
        int isum[NB][16];
#pragma unroll
        for (int i = 0; i < NB; i++)
#pragma unroll
            for (int v = 0; v < 16; v++) isum[i][v] = 0;
        const gs_i16 zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        // the eight 6-bit scales and mins, a byte each (get_scale_min_k4, crates/ojas-formats/src/gguf.rs:1132-1140)
        const uint sc_lo = r.hdr.y & 0x3F3F3F3Fu, mn_lo = r.hdr.z & 0x3F3F3F3Fu;
        const uint sc_hi = (r.hdr.w & 0x0F0F0F0Fu) | ((r.hdr.y >> 2) & 0x30303030u);
        const uint mn_hi = ((r.hdr.w >> 4) & 0x0F0F0F0Fu) | ((r.hdr.z >> 2) & 0x30303030u);
        // sub-block j, half h: the codes of positions 16 h + 8 kg .. of chunk j / 2 (low or high nibbles) under fifth bit j
        auto codes = [&](int j, int h) -> long {
            const uint2 p = r.qs[j >> 1][h];
            const uint n0 = (j & 1) ? (p.x >> 4) & 0x0F0F0F0Fu : p.x & 0x0F0F0F0Fu;
            const uint n1 = (j & 1) ? (p.y >> 4) & 0x0F0F0F0Fu : p.y & 0x0F0F0F0Fu;
            const uint b0 = j < 4 ? (r.qh[h].x << (4 - j)) & 0x10101010u : (r.qh[h].x >> (j - 4)) & 0x10101010u;
            const uint b1 = j < 4 ? (r.qh[h].y << (4 - j)) & 0x10101010u : (r.qh[h].y >> (j - 4)) & 0x10101010u;
            return gq_pack(n0 | b0, n1 | b1);
        };
        auto tokens = [&](int j, int h, int i) -> long {
            return *(const long*)(xa + (uint)i * 32u * GS_STRIDE + 32u * (uint)j + 16u * (uint)h);
        };
        // the next sub-block's operands are fetched and built under this one's matrix instructions
        long B[2] = {codes(0, 0), codes(0, 1)};
        long A[2][2] = {{tokens(0, 0, 0), NB == 2 ? tokens(0, 0, 1) : 0}, {tokens(0, 1, 0), NB == 2 ? tokens(0, 1, 1) : 0}};
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int s = (int)(((j < 4 ? sc_lo : sc_hi) >> (8 * (j & 3))) & 0xFFu);
            // (one instruction over all 32 positions of the sub-block: a lane's sixteen are 8 kg .. and 16 + 8 kg ..)
            gs_i16 D[NB];
            const gq_i4 Bj = {(int)B[0], (int)(B[0] >> 32), (int)B[1], (int)(B[1] >> 32)};
#pragma unroll
            for (int i = 0; i < NB; i++) {
                const gq_i4 Aj = {(int)A[0][i], (int)(A[0][i] >> 32), (int)A[1][i], (int)(A[1][i] >> 32)};
                D[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(Aj, Bj, zero, 0, 0, 0);
            }
            if (j < 7) {
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    B[h] = codes(j + 1, h);
                    A[h][0] = tokens(j + 1, h, 0);
                    if (NB == 2) A[h][1] = tokens(j + 1, h, 1);
                }
            }
#pragma unroll
            for (int i = 0; i < NB; i++)
#pragma unroll
                for (int v = 0; v < 16; v++) isum[i][v] = gs_pin(isum[i][v] + __mul24(s, D[i][v]));
            __builtin_amdgcn_sched_barrier(0);
        }
        // sum_j m_j bsum_j, bsum = 64 hi + lo: positions 0..7 of A carry the lo parts, 8..15 the hi parts, B the mins twice:
        // D1 = sum m lo + sum m hi; with the lo half of A blanked D2 = sum m hi; the term is D1 + 63 D2
        const long Bm = gq_pack(mn_lo, mn_hi);
        const long km = kg ? -1l : 0l;
        const float d = f16_bits_to_f32(r.hdr.x & 0xFFFFu), dmin = f16_bits_to_f32(r.hdr.x >> 16);
#pragma unroll
        for (int i = 0; i < NB; i++) {
            const long A1 = *(const long*)(st + GS_BS + (tok0 + 32u * (uint)i + fr) * 16u + 8u * kg);
            const gs_i16 D1 = __builtin_amdgcn_mfma_i32_32x32x16_i8(A1, Bm, zero, 0, 0, 0);
            const gs_i16 D2 = __builtin_amdgcn_mfma_i32_32x32x16_i8(A1 & km, Bm, zero, 0, 0, 0);
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const float4 x4 = *(const float4*)(sx + 32 * i + 8 * g);
                const float xv[4] = {x4.x, x4.y, x4.z, x4.w};
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int v = 4 * g + e;
                    const float inner = __fmaf_rn(-dmin, (float)(D1[v] + 63 * D2[v]), __fmul_rn(d, (float)isum[i][v]));
                    acc[i][v] = __fmaf_rn(xv[e], inner, acc[i][v]);
                }
            }
        }
    }
};

// which row of xq / xs / y token m of the launch is: itself, or (grouped expert products) an entry of a list
struct GsDense {
    __device__ __forceinline__ uint row(uint m) const { return m; }
};
struct GsList {
    const uint* lst;
    uint last;
    __device__ __forceinline__ uint row(uint m) const { return min(lst[m], last); }
};
template <class F, bool SPLIT, class TM = GsDense>
__device__ __forceinline__ void gemm_q8k_gs_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                                 const uchar* __restrict__ w, float* __restrict__ y, uint K, uint N, uint M,
                                                 uint ACC, uchar* lds, float* part = nullptr, uint* cnt = nullptr,
                                                 uint nsplit = 1u, const TM tm = TM(), uint ty = blockIdx.y) {
    const uint tid = threadIdx.x, lane = tid & 63u;
    const uint wave = (uint)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint nsb = K >> 8;
    const uint per = SPLIT ? (nsb + nsplit - 1u) / nsplit : nsb;
    const uint sb0 = SPLIT ? blockIdx.z * per : 0u, sb1 = SPLIT ? min(nsb, sb0 + per) : nsb;
    if (SPLIT && sb0 >= sb1) return;                      // (the host launches only slices that hold a super-block)
    constexpr uint TPG = 64u, RPG = 128u;                     // tokens and rows per workgroup
    const uint m0 = ty * TPG, fr = lane & 31u, kg = lane >> 5;
    const uint row = min(blockIdx.x * RPG + 32u * wave + fr, N - 1u);
    const uint tok0 = 0u;
    // 32-token blocks that hold tokens: the last token tile may need only the first
    const uint nblk = M - m0 > 32u ? 2u : 1u;
    const uchar* wr = w + (size_t)row * nsb * F::BYTES;

    // staging: thread -> chunk tid % 16 (16 bytes) of tokens tid / 16 + 16 p, p = 0 .. 3
    constexpr int NP = 4;
    const uint s_tok = tid >> 4, s_ch = tid & 15u;
    uint4 tv[NP];
    float tsx = 0.0f;
    // the rows of this thread's tokens (one lookup per tile, not per super-block)
    uint trow[NP];
#pragma unroll
    for (int p = 0; p < NP; p++) trow[p] = tm.row(min(m0 + s_tok + 16u * (uint)p, M - 1u));
    const uint xrow = tm.row(min(m0 + tid, M - 1u));
    auto fetch = [&](uint sb) {
#pragma unroll
        for (int p = 0; p < NP; p++) {
            const uint m = m0 + s_tok + 16u * (uint)p;
            tv[p] = make_uint4(0u, 0u, 0u, 0u);
            if (m < M) tv[p] = *(const uint4*)(xq + (size_t)trow[p] * K + (size_t)sb * 256u + s_ch * 16u);
        }
        if (tid < TPG) tsx = m0 + tid < M ? xs[(size_t)xrow * nsb + sb] : 0.0f;
    };
    auto put = [&](uchar* st) {
#pragma unroll
        for (int p = 0; p < NP; p++) {
            uchar* o = st + (s_tok + 16u * (uint)p) * GS_STRIDE + s_ch * 16u;
            *(uint2*)o = make_uint2(tv[p].x, tv[p].y);
            *(uint2*)(o + 8) = make_uint2(tv[p].z, tv[p].w);
            if (F::BSUMS) {
                // half a sub-block per thread; its neighbour holds the other half
                int s = dot4_i8(tv[p].x, 0x01010101u, 0);
                s = dot4_i8(tv[p].y, 0x01010101u, s);
                s = dot4_i8(tv[p].z, 0x01010101u, s);
                s = dot4_i8(tv[p].w, 0x01010101u, s);
                s += dpp_i32<OJK_DPP_QUAD_XOR1>(s);
                if (!(s_ch & 1u)) {
                    uchar* b = st + GS_BS + (s_tok + 16u * (uint)p) * 16u + (s_ch >> 1);
                    b[0] = (uchar)(s & 63);
                    b[8] = (uchar)(s >> 6);
                }
            }
        }
        if (tid < TPG) ((float*)(st + GS_SX))[tid] = tsx;
    };

    float acc[2][16];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[i][v] = 0.0f;

    fetch(sb0);
    typename F::Raw nx = F::load(wr + (size_t)sb0 * F::BYTES, kg);
    put(lds);
    __syncthreads();
    for (uint sb = sb0; sb < sb1; sb++) {
        const typename F::Raw cur = nx;
        const uint nb = min(sb + 1u, sb1 - 1u);
        nx = F::load(wr + (size_t)nb * F::BYTES, kg);
        fetch(nb);
        const uchar* st = lds + ((sb - sb0) & 1u) * GS_STAGE;
        if (nblk == 2u) F::template superblock<2>(cur, st, tok0, fr, kg, acc);
        else F::template superblock<1>(cur, st, tok0, fr, kg, acc);
        put(lds + (((sb - sb0) & 1u) ^ 1u) * GS_STAGE);
        __syncthreads();
    }

    if (SPLIT) {
        // partial tiles out as the registers hold them ([pair][thread]), written through and read from behind the L2
        // (a tile's slices run on different XCDs); the stores are awaited by instruction before the slice is counted
        typedef unsigned long long u64;
        const uint ns_eff = (nsb + per - 1u) / per;
        const uint tile = blockIdx.y * gridDim.x + blockIdx.x;
        u64* const mine = (u64*)part + ((size_t)tile * ns_eff + blockIdx.z) * 16u * 256u + tid;
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
            for (int h = 0; h < 8; h++)
                __hip_atomic_store(mine + (size_t)(i * 8 + h) * 256u,
                                   (u64)__float_as_uint(acc[i][2 * h]) | ((u64)__float_as_uint(acc[i][2 * h + 1]) << 32),
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __syncthreads();
        if (tid == 0u) *(volatile uint*)lds = atomicAdd(cnt + tile, 1u);
        __syncthreads();
        if ((uint)__builtin_amdgcn_readfirstlane((int)*(volatile uint*)lds) != ns_eff - 1u) return;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        const u64* const all = (const u64*)part + (size_t)tile * ns_eff * 16u * 256u + tid;
        for (uint s0 = 0; s0 < ns_eff; s0 += 2u) {
            u64 v[2][16];
#pragma unroll
            for (int q = 0; q < 2; q++) {
                const uint sl = min(s0 + (uint)q, ns_eff - 1u);
#pragma unroll
                for (int i = 0; i < 16; i++)
                    v[q][i] = __hip_atomic_load(all + ((size_t)sl * 16u + (uint)i) * 256u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            }
#pragma unroll
            for (int q = 0; q < 2; q++) {
                if (s0 + (uint)q < ns_eff) {
                    const bool first = s0 + (uint)q == 0u;
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const float a = __uint_as_float((uint)v[q][i]), b = __uint_as_float((uint)(v[q][i] >> 32));
                        acc[i / 8][2 * (i % 8)] = first ? a : acc[i / 8][2 * (i % 8)] + a;
                        acc[i / 8][2 * (i % 8) + 1] = first ? b : acc[i / 8][2 * (i % 8) + 1] + b;
                    }
                }
            }
        }
        if (tid == 0u) cnt[tile] = 0u;                               // ready for the next launch
    }
    // D register v of block i: token 32 i + 8 (v / 4) + 4 kg + v % 4, row fr
    const uint n = blockIdx.x * RPG + 32u * wave + fr;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
            const uint t = m0 + tok0 + 32u * (uint)i + 8u * (uint)(v >> 2) + 4u * kg + (uint)(v & 3);
            if (t < M && n < N) {
                float* o = y + (size_t)tm.row(t) * N + n;
                *o = ACC ? *o + acc[i][v] : acc[i][v];
            }
        }
}

#define GEMM_Q8K_GS(FMT, F)                                                                                              \
    extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))                         \
    gemm_q8k_##FMT##_gs(const signed char* xq, const float* xs, const uchar* w, float* y, uint K, uint N, uint M, uint ACC) { \
        __shared__ __attribute__((aligned(16))) uchar lds_gs[2 * GS_STAGE];                                              \
        gemm_q8k_gs_body<F, false>(xq, xs, w, y, K, N, M, ACC, lds_gs);                                                  \
    }                                                                                                                    \
    extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))                         \
    gemm_q8k_##FMT##_gs_sr(const signed char* xq, const float* xs, const uchar* w, float* y, float* part, uint* cnt,     \
                           uint K, uint N, uint M, uint ACC, uint NSPLIT) {                                              \
        __shared__ __attribute__((aligned(16))) uchar lds_gs[2 * GS_STAGE];                                              \
        gemm_q8k_gs_body<F, true>(xq, xs, w, y, K, N, M, ACC, lds_gs, part, cnt, NSPLIT);                                \
    }
GEMM_Q8K_GS(q6k, GsQ6K)
GEMM_Q8K_GS(q5k, GsQ5K)

// The same tile over grouped expert products (the down projection of a mixture-of-experts layer whose down tensors are
// Q6_K / Q5_K): expert e = blockIdx.z owns rows e N .. of `wd` and the assignments list[offsets[e] .. offsets[e + 1]);
// token tiles blockIdx.y, + gridDim.y, .. of them (workgroups past the expert's count leave at once), results unweighted
// into dv[a][n].
//   moe_down_{q6k,q5k}_gs(aq, as, wd, dv, offsets, list, K, N, NA)     grid [ceil(N / 128), 1 .. ceil(T / 64), E] x 256
#define MOE_DOWN_GS(FMT, F)                                                                                              \
    extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))                         \
    moe_down_##FMT##_gs(const signed char* aq, const float* as_, const uchar* wd, float* dv, const uint* offsets,        \
                        const uint* list, uint K, uint N, uint NA) {                                                     \
        __shared__ __attribute__((aligned(16))) uchar lds_gs[2 * GS_STAGE];                                              \
        const uint e = blockIdx.z;                                                                                       \
        const uint a0 = min(offsets[e], NA), a1 = min(offsets[e + 1], NA);                                               \
        if (a0 >= a1) return;                                                                                            \
        GsList tm;                                                                                                       \
        tm.lst = list + a0;                                                                                              \
        tm.last = NA - 1u;                                                                                               \
        for (uint ty = blockIdx.y; ty * 64u < a1 - a0; ty += gridDim.y) {                                                \
            gemm_q8k_gs_body<F, false, GsList>(aq, as_, wd + (size_t)e * N * (K >> 8) * F::BYTES, dv, K, N, a1 - a0, 0u, \
                                               lds_gs, nullptr, nullptr, 1u, tm, ty);                                    \
            __syncthreads();                                                                                             \
        }                                                                                                                \
    }
MOE_DOWN_GS(q6k, GsQ6K)
MOE_DOWN_GS(q5k, GsQ5K)
