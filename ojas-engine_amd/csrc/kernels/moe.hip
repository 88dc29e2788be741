// Family "moe": router and grouped expert FFN on raw Q4_K expert tensors.
//
// Semantics (reference: router crates/ojas-cuda/src/kernels/moe.rs:45-70; expert FFN
// crates/ojas-cpu/src/cpu_glm.rs:551-582, batched per-assignment GPU form
// crates/ojas-metal/src/kernels/moe.rs:199-272):
//   idx, wgt = top-KSEL of softmax(logits), lowest index wins ties, weights renormalised
//   for every assignment a = (token t, slot j), e = idx[a]:
//       act[a] = silu(Wg_e x_t) * (Wu_e x_t);   dv[a] = Wd_e act[a]
//   y[t] (+)= sum_j wgt[t][j] * dv[t*KSEL + j]           (slot order, f32)
// with every matvec in the CPU reference's arithmetic (activations quantized per 256 by quant_q8k,
// integer dots, crates/ojas-cpu/src/cpu_math.rs:539-635).
//
// The reference launches one workgroup column per assignment and leans on the cache for experts
// shared by several tokens.  Here assignments are grouped by expert first (moe_group: counting
// sort -> per-expert offsets + assignment list), and one launch per projection walks the
// experts: a wave loads its rows of expert e once into registers and runs them against every
// token routed to e, so an expert's bytes cross HBM once however many tokens chose it.
//
//   moe_topk(lg, idx, wgt, E, KSEL)                          one token, 1 x 64 threads
//   moe_topk_m(lg, idx, wgt, E, KSEL)                        grid = tokens
//   moe_group(idx, counts, offsets, list, NA, E)             1 x 256 threads; NA = tokens*KSEL
//   moe_gu_q4k_m(xq, xs, wg, wu, act, offsets, list, K, N, KSEL, NA)   grid (ceil(N/8), E)
//   moe_down_{q4k,q5k}_m(aq, as, wd, dv, offsets, list, K, N, NA)      grid (ceil(N/16), E); ceil(N/32) for K <= 1024
//   moe_combine(dv, wgt, y, T, KSEL, D, ACC)                 grid ceil(T*D/256)
//   moe_gu_q4k_dec(x, wg, wu, act, idx, K, N, KSEL, NA, E)   grid (ceil(N/8), NA): few tokens, f32 in
//   moe_gu_q4k_decr(x, wg, wu, act, lg, idx, wgt, K, N, KSEL, NA, E)  the same with the router inside (writes idx, wgt)
//   moe_down_{q4k,q5k}_dec(act, wd, idx, wgt, y, K, N, KSEL, E, ACC)  grid (ceil(N/8), T): down + weighted sum
//   moe_gu_q4k_slots(x, arena_g, arena_u, act, off_g, off_u, K, N, KSEL, NA, LIM_G, LIM_U)   the decode form over
//   moe_down_q4k_slots(act, arena, off_d, wgt, y, K, N, KSEL, LIM, ACC)                     streamed experts (u64 byte offsets)
//   moe_gu_q4k_mm / moe_down_q4k_mm, moe_gu_q4k_mt / moe_down_q4k_mt (same arguments as the _m entries)
//                                                            grid (ceil(N/16), E): the int8 matrix-core form
#include "ojk_common.h"
#include "ojk_q4k_dot.h"
#include "ojk_gq.h"
#include "ojk_moe_rows.h"

// ------------------------------------------------------------------ router
template <int NI>
__device__ __forceinline__ void moe_topk_lanes(const float* __restrict__ lg, uint* __restrict__ idx,
                                               float* __restrict__ wgt, uint E, uint KSEL) {
    // one wave per token; lane l owns experts l, l+64, ... (E <= 64 NI)
    const uint lane = threadIdx.x & 63u;
    float p[NI];
    float mx = -3.4028235e38f;
#pragma unroll
    for (int i = 0; i < NI; i++) {
        uint e = lane + 64u * i;
        p[i] = e < E ? lg[e] : -3.4028235e38f;
        mx = fmaxf(mx, p[i]);
    }
    mx = wave_max(mx);
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < NI; i++) {
        uint e = lane + 64u * i;
        p[i] = e < E ? expf(p[i] - mx) : -1.0f;
        if (e < E) sum += p[i];
    }
    sum = wave_sum(sum);
#pragma unroll
    for (int i = 0; i < NI; i++)
        if (lane + 64u * i < E) p[i] = p[i] / sum;
    float wsum = 0.0f, mine = 0.0f;
    uint mine_idx = 0;
    for (uint j = 0; j < KSEL; j++) {
        float bv = -1.0f;
        uint bi = 0xFFFFFFFFu;
#pragma unroll
        for (int i = 0; i < NI; i++) {  // ascending expert index within the lane: '>' keeps the lowest
            if (p[i] > bv) { bv = p[i]; bi = lane + 64u * i; }
        }
        float m2 = wave_max(bv);
        // lowest index among the lanes holding the maximum: an expert's index is lane + 64 i, so the lowest i with any
        // such lane decides, and within it the lowest lane — one vote per i and scalar bit scans instead of a second
        // reduction across the wave
        uint win = 0xFFFFFFFFu;
#pragma unroll
        for (int i = NI - 1; i >= 0; i--) {
            const unsigned long long vote = __ballot(bv == m2 && bi == lane + 64u * (uint)i);
            if (vote) win = (uint)__builtin_ctzll(vote) + 64u * (uint)i;
        }
        wsum += m2;
        if (lane == j) { mine = m2; mine_idx = win; }
#pragma unroll
        for (int i = 0; i < NI; i++)
            if (lane + 64u * i == win) p[i] = -1.0f;
    }
    if (lane < KSEL) {
        idx[lane] = mine_idx;
        wgt[lane] = mine / wsum;
    }
}

__device__ __forceinline__ void moe_topk_body(const float* __restrict__ lg, uint* __restrict__ idx,
                                              float* __restrict__ wgt, uint E, uint KSEL) {
    if (E <= 128u) moe_topk_lanes<2>(lg, idx, wgt, E, KSEL);
    else if (E <= 256u) moe_topk_lanes<4>(lg, idx, wgt, E, KSEL);
    else moe_topk_lanes<16>(lg, idx, wgt, E, KSEL);
}

extern "C" __global__ void __launch_bounds__(64)
moe_topk(const float* lg, uint* idx, float* wgt, uint E, uint KSEL) {
    moe_topk_body(lg, idx, wgt, E, KSEL);
}
extern "C" __global__ void __launch_bounds__(64)
moe_topk_m(const float* lg, uint* idx, float* wgt, uint E, uint KSEL) {
    const size_t t = blockIdx.x;
    moe_topk_body(lg + t * E, idx + t * KSEL, wgt + t * KSEL, E, KSEL);
}

// ---- the reference's other routers (Metal twins crates/ojas-metal/src/kernels/moe.rs:130-150, :531-551) ----
//   moe_topk_nonorm(lg, idx, wgt, E, KSEL)                     DeepSeek-V2: softmax, top-KSEL, the raw probabilities
//   moe_topk_v3(lg, bias, idx, wgt, E, KSEL, RSCALE, NORM)     DeepSeek-V3 / GLM: s = sigmoid(logit); experts chosen by
//       s + bias (strict '>', lowest index wins ties); weight = s of the chosen, times 1 / (their sum) when NORM and the
//       sum is positive, times the routed scaling factor (RSCALE: its f32 bits) — crates/ojas-cpu/src/cpu_glm.rs:526-548
// grid [tokens,1,1] x 64: token t reads lg + t E and writes idx / wgt + t KSEL (one token: grid [1,1,1]).
template <int NI, bool V3>
__device__ __forceinline__ void moe_topk_alt_lanes(const float* __restrict__ lg, const float* __restrict__ bias,
                                                   uint* __restrict__ idx, float* __restrict__ wgt, uint E, uint KSEL,
                                                   float rscale, uint norm) {
    const uint lane = threadIdx.x & 63u;
    float ch[NI], val[NI];      // what the experts are chosen by; what a chosen expert's weight is made of
    float sum = 1.0f;
    if (V3) {
#pragma unroll
        for (int i = 0; i < NI; i++) {
            const uint e = lane + 64u * i;
            const float sg = e < E ? 1.0f / (1.0f + expf(-lg[e])) : 0.0f;
            val[i] = sg;
            ch[i] = e < E ? sg + bias[e] : -3.4028235e38f;
        }
    } else {
        float mx = -1e30f;
#pragma unroll
        for (int i = 0; i < NI; i++) {
            const uint e = lane + 64u * i;
            ch[i] = e < E ? lg[e] : -3.4028235e38f;
            if (e < E) mx = fmaxf(mx, ch[i]);
        }
        mx = wave_max(mx);
        sum = 0.0f;
#pragma unroll
        for (int i = 0; i < NI; i++) {
            const uint e = lane + 64u * i;
            ch[i] = e < E ? expf(ch[i] - mx) : -3.4028235e38f;
            val[i] = ch[i];
            if (e < E) sum += ch[i];
        }
        sum = wave_sum(sum);
    }
    float wsum = 0.0f, mine = 0.0f;
    uint mine_idx = 0;
    for (uint j = 0; j < KSEL; j++) {
        float bv = V3 ? -1e30f : -1.0f, bval = 0.0f;
        uint bi = 0xFFFFFFFFu;
#pragma unroll
        for (int i = 0; i < NI; i++)
            if (ch[i] > bv) { bv = ch[i]; bval = val[i]; bi = lane + 64u * i; }
        const float m2 = wave_max(bv);
        uint cand = (bv == m2 && bi != 0xFFFFFFFFu) ? bi : 0xFFFFFFFFu;
        cand = min(cand, (uint)dpp_i32<OJK_DPP_QUAD_XOR1>((int)cand));
        cand = min(cand, (uint)dpp_i32<OJK_DPP_QUAD_XOR2>((int)cand));
        cand = min(cand, (uint)dpp_i32<OJK_DPP_ROW_HALF_MIRROR>((int)cand));
        cand = min(cand, (uint)dpp_i32<OJK_DPP_ROW_MIRROR>((int)cand));
        const uint c0 = (uint)__builtin_amdgcn_readlane((int)cand, 0), c1 = (uint)__builtin_amdgcn_readlane((int)cand, 16);
        const uint c2 = (uint)__builtin_amdgcn_readlane((int)cand, 32), c3 = (uint)__builtin_amdgcn_readlane((int)cand, 48);
        const uint win = min(min(c0, c1), min(c2, c3));
        // the winner's value (its lane holds it): all lanes learn it
        const uint wl = win & 63u;
        float wv = 0.0f;
#pragma unroll
        for (int i = 0; i < NI; i++)
            if (lane + 64u * i == win) wv = val[i];
        wv = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wv), (int)__builtin_amdgcn_readfirstlane((int)wl)));
        (void)bval;
        wsum += wv;
        if (lane == j) { mine = wv; mine_idx = win; }
#pragma unroll
        for (int i = 0; i < NI; i++)
            if (lane + 64u * i == win) ch[i] = V3 ? -1e30f : -1.0f;
    }
    if (lane < KSEL) {
        idx[lane] = mine_idx;
        if (V3) {
            const float inv = (norm != 0u && wsum > 0.0f) ? 1.0f / wsum : 1.0f;
            wgt[lane] = mine * inv * rscale;
        } else {
            wgt[lane] = mine / sum;
        }
    }
}

extern "C" __global__ void __launch_bounds__(64)
moe_topk_nonorm(const float* lg, uint* idx, float* wgt, uint E, uint KSEL) {
    const size_t t = blockIdx.x;
    if (E <= 128u) moe_topk_alt_lanes<2, false>(lg + t * E, nullptr, idx + t * KSEL, wgt + t * KSEL, E, KSEL, 1.0f, 0u);
    else if (E <= 256u) moe_topk_alt_lanes<4, false>(lg + t * E, nullptr, idx + t * KSEL, wgt + t * KSEL, E, KSEL, 1.0f, 0u);
    else moe_topk_alt_lanes<16, false>(lg + t * E, nullptr, idx + t * KSEL, wgt + t * KSEL, E, KSEL, 1.0f, 0u);
}
extern "C" __global__ void __launch_bounds__(64)
moe_topk_v3(const float* lg, const float* bias, uint* idx, float* wgt, uint E, uint KSEL, uint RSCALE, uint NORM) {
    const size_t t = blockIdx.x;
    const float rs = __uint_as_float(RSCALE);
    if (E <= 128u) moe_topk_alt_lanes<2, true>(lg + t * E, bias, idx + t * KSEL, wgt + t * KSEL, E, KSEL, rs, NORM);
    else if (E <= 256u) moe_topk_alt_lanes<4, true>(lg + t * E, bias, idx + t * KSEL, wgt + t * KSEL, E, KSEL, rs, NORM);
    else moe_topk_alt_lanes<16, true>(lg + t * E, bias, idx + t * KSEL, wgt + t * KSEL, E, KSEL, rs, NORM);
}

// ------------------------------------------------------------------ grouping
// Counting sort of the NA assignments by expert: counts[E], offsets[E+1], list[NA] (assignment
// ids, expert-major; the order inside an expert's group is arbitrary and has no effect on the
// results, which are stored per assignment).  One workgroup; E <= 1024.
__device__ __forceinline__ void moe_group_body(const uint* __restrict__ idx, uint* __restrict__ counts, uint* __restrict__ offsets,
                                               uint* __restrict__ list, uint NA, uint E, uint* cnt, uint* off) {
    const uint tid = threadIdx.x;
    for (uint e = tid; e < E; e += 256u) cnt[e] = 0u;
    __syncthreads();
    // (eight loads in flight per thread: one at a time, each pass over the assignments cost a round trip to memory per
    // 256 of them — 8 us per pass at 2048)
    for (uint a0 = tid; a0 < NA; a0 += 8u * 256u) {
        uint e[8];
#pragma unroll
        for (int u = 0; u < 8; u++) e[u] = a0 + (uint)u * 256u < NA ? idx[a0 + (uint)u * 256u] : 0xFFFFFFFFu;
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (e[u] < E) atomicAdd(&cnt[e[u]], 1u);
    }
    __syncthreads();
    {
        // exclusive prefix sums of the counts: a thread takes four consecutive experts (E <= 1024), the threads' totals
        // are scanned across the wave by shuffles and across the four waves through off[1024] .. (free until the end)
        const uint lane = tid & 63u, wv = tid >> 6;
        uint c[4], local = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            c[i] = 4u * tid + (uint)i < E ? cnt[4u * tid + (uint)i] : 0u;
            local += c[i];
        }
        uint incl = local;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint up = (uint)__shfl_up((int)incl, d);
            if (lane >= (uint)d) incl += up;
        }
        __shared__ uint wtot[4];
        if (lane == 63u) wtot[wv] = incl;
        __syncthreads();
        uint base = 0;
        for (uint w = 0; w < wv; w++) base += wtot[w];
        uint run = base + incl - local;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if (4u * tid + (uint)i < E) off[4u * tid + (uint)i] = run;
            run += c[i];
        }
        if (tid == 255u) off[E] = run;      // thread 255 ends at the grand total
    }
    __syncthreads();
    for (uint e = tid; e <= E; e += 256u) {
        offsets[e] = off[e];
        if (e < E) counts[e] = cnt[e];
    }
    for (uint e = tid; e < E; e += 256u) cnt[e] = 0u;  // reused as the per-expert cursor
    __syncthreads();
    for (uint a0 = tid; a0 < NA; a0 += 8u * 256u) {
        uint e[8];
#pragma unroll
        for (int u = 0; u < 8; u++) e[u] = a0 + (uint)u * 256u < NA ? idx[a0 + (uint)u * 256u] : 0xFFFFFFFFu;
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (e[u] < E) list[off[e[u]] + atomicAdd(&cnt[e[u]], 1u)] = a0 + (uint)u * 256u;
    }
}
extern "C" __global__ void __launch_bounds__(256)
moe_group(const uint* __restrict__ idx, uint* __restrict__ counts, uint* __restrict__ offsets,
          uint* __restrict__ list, uint NA, uint E) {
    __shared__ uint cnt[1024];
    __shared__ uint off[1025];
    moe_group_body(idx, counts, offsets, list, NA, E, cnt, off);
}

// ------------------------------------------------------------------ grouped gate / up
// Block (rb, e): 4 waves x 2 rows = 8 rows of expert e's gate and up.  K must be a multiple of
// 256; a wave walks K in steps of 8 super-blocks (one step for the usual hidden sizes).
extern "C" __global__ void __launch_bounds__(256)
moe_gu_q4k_m(const signed char* __restrict__ xq, const float* __restrict__ xs, const uchar* __restrict__ wg,
             const uchar* __restrict__ wu, float* __restrict__ act, const uint* __restrict__ offsets,
             const uint* __restrict__ list, uint K, uint N, uint KSEL, uint NA) {
    const uint e = blockIdx.y;
    const uint a0 = min(offsets[e], NA), a1 = min(offsets[e + 1], NA);
    if (a0 >= a1) return;
    const uint lane = threadIdx.x & 63u;
    const uint row0 = (blockIdx.x * 4u + (threadIdx.x >> 6)) * 2u;
    if (row0 >= N) return;
    const uint nsb = K >> 8, g = lane >> 3, l = lane & 7u, c = l >> 1;
    const size_t rb = (size_t)nsb * Q4K_BYTES;
    const uchar* g0 = wg + ((size_t)e * N + row0) * rb;
    const uchar* u0 = wu + ((size_t)e * N + row0) * rb;
    const bool two = row0 + 1u < N;
    const size_t r1 = two ? rb : 0;
    if (nsb <= 8u) {
        // the whole row fits one step: weights stay in registers across the expert's tokens
        const bool on = g < nsb;
        const size_t o = (size_t)(on ? g : 0u) * Q4K_BYTES;
        uint4 hg0 = *(const uint4*)(g0 + o), qg0 = *(const uint4*)(g0 + o + 16u + l * 16u);
        uint4 hg1 = *(const uint4*)(g0 + r1 + o), qg1 = *(const uint4*)(g0 + r1 + o + 16u + l * 16u);
        uint4 hu0 = *(const uint4*)(u0 + o), qu0 = *(const uint4*)(u0 + o + 16u + l * 16u);
        uint4 hu1 = *(const uint4*)(u0 + r1 + o), qu1 = *(const uint4*)(u0 + r1 + o + 16u + l * 16u);
        for (uint i = a0; i < a1; i++) {
            const uint a = min(list[i], NA - 1u), t = a / KSEL;
            Q4kFrag f = q4k_load_frag(xq + (size_t)t * nsb * 256u, xs + (size_t)t * nsb, on ? g : 0u, l);
            // (lanes past the row's last super-block multiply by a zero scale: a product of zero, and no branch around
            // each of the four dots)
            f.sx = on ? f.sx : 0.0f;
            float vg0 = q4k_lane_dot(hg0, qg0, c, f), vg1 = q4k_lane_dot(hg1, qg1, c, f);
            float vu0 = q4k_lane_dot(hu0, qu0, c, f), vu1 = q4k_lane_dot(hu1, qu1, c, f);
            // the four sums in one pass: lanes 0 / 1 end with the gate sums of the two rows, lanes 2 / 3 with the up sums
            const float tot = wave_sum4(vg0, vg1, vu0, vu1, lane);
            const float upv = dpp_f32<OJK_DPP_QUAD_XOR2>(tot);
            if (lane < (two ? 2u : 1u)) act[(size_t)a * N + row0 + lane] = (tot / (1.0f + expf(-tot))) * upv;
        }
    } else {
        for (uint i = a0; i < a1; i++) {
            const uint a = min(list[i], NA - 1u), t = a / KSEL;
            float vg0 = 0.0f, vg1 = 0.0f, vu0 = 0.0f, vu1 = 0.0f;
            for (uint sb = g; sb < nsb; sb += 8u) {
                const size_t o = (size_t)sb * Q4K_BYTES;
                Q4kFrag f = q4k_load_frag(xq + (size_t)t * nsb * 256u, xs + (size_t)t * nsb, sb, l);
                vg0 += q4k_lane_dot(*(const uint4*)(g0 + o), *(const uint4*)(g0 + o + 16u + l * 16u), c, f);
                vg1 += q4k_lane_dot(*(const uint4*)(g0 + r1 + o), *(const uint4*)(g0 + r1 + o + 16u + l * 16u), c, f);
                vu0 += q4k_lane_dot(*(const uint4*)(u0 + o), *(const uint4*)(u0 + o + 16u + l * 16u), c, f);
                vu1 += q4k_lane_dot(*(const uint4*)(u0 + r1 + o), *(const uint4*)(u0 + r1 + o + 16u + l * 16u), c, f);
            }
            const float tot = wave_sum4(vg0, vg1, vu0, vu1, lane);
            const float upv = dpp_f32<OJK_DPP_QUAD_XOR2>(tot);
            if (lane < (two ? 2u : 1u)) act[(size_t)a * N + row0 + lane] = (tot / (1.0f + expf(-tot))) * upv;
        }
    }
}

// ------------------------------------------------------------------ grouped down
// Block (rb, e): 4 waves x 4 rows = 16 rows of expert e's down projection, against the quantized
// act of every assignment routed to e.  dv[a][n] holds the unweighted result.
template <class W>
__device__ __forceinline__ void moe_down_m_body(const signed char* __restrict__ aq, const float* __restrict__ as_,
                                                const uchar* __restrict__ wd, float* __restrict__ dv,
                                                const uint* __restrict__ offsets, const uint* __restrict__ list,
                                                uint K, uint N, uint NA) {
    const uint e = blockIdx.y;
    const uint a0 = min(offsets[e], NA), a1 = min(offsets[e + 1], NA);
    if (a0 >= a1) return;
    const uint lane = threadIdx.x & 63u;
    const uint nsb = K >> 8, g = lane >> 3, l = lane & 7u, c = l >> 1;
    const size_t rb = (size_t)nsb * W::BYTES;
    if (nsb <= 4u) {
        // A short row (an expert's down projection: 768 = 3 super-blocks) leaves most of a wave idle in
        // the layout below.  Here the wave's halves take different rows: 8 rows per wave, 32 per
        // workgroup, and a half's two 16-lane sums are added as wave_sum adds them.
        const uint hf = lane >> 5, G = g & 3u;
        const uint rowh = (blockIdx.x * 4u + (threadIdx.x >> 6)) * 8u + hf * 4u;     // this half's first row
        const bool on = G < nsb;
        const uchar* wh = wd + ((size_t)e * N + min(rowh, N - 1u)) * rb + (size_t)(on ? G : 0u) * W::BYTES;
        W wr[4];
#pragma unroll
        for (int r = 0; r < 4; r++) wr[r].load(wh + (size_t)min((uint)r, N - 1u - min(rowh, N - 1u)) * rb, l);
        for (uint i = a0; i < a1; i++) {
            const uint a = min(list[i], NA - 1u);
            Q4kFrag f = q4k_load_frag(aq + (size_t)a * nsb * 256u, as_ + (size_t)a * nsb, on ? G : 0u, l);
            f.sx = on ? f.sx : 0.0f;        // lanes without a super-block of the row: products of zero, no branches
            // the half's four rows in one pass: lane j of each row of 16 gets row j's 16-lane sum, the half's two
            // such sums are added as wave_sum adds them
            float v = row16_sum4(wr[0].dot(c, f), wr[1].dot(c, f), wr[2].dot(c, f), wr[3].dot(c, f), lane);
            v += __shfl_xor(v, 16);
            if ((lane & 31u) < 4u && rowh + (lane & 3u) < N) dv[(size_t)a * N + rowh + (lane & 3u)] = v;
        }
        return;
    }
    const uint row0 = (blockIdx.x * 4u + (threadIdx.x >> 6)) * 4u;
    if (row0 >= N) return;
    const uchar* w0 = wd + ((size_t)e * N + row0) * rb;
    if (nsb <= 8u) {
        const bool on = g < nsb;
        const size_t o = (size_t)(on ? g : 0u) * W::BYTES;
        W wr[4];
#pragma unroll
        for (int r = 0; r < 4; r++) wr[r].load(w0 + (size_t)min((uint)r, N - 1u - row0) * rb + o, l);
        for (uint i = a0; i < a1; i++) {
            const uint a = min(list[i], NA - 1u);
            Q4kFrag f = q4k_load_frag(aq + (size_t)a * nsb * 256u, as_ + (size_t)a * nsb, on ? g : 0u, l);
            f.sx = on ? f.sx : 0.0f;
            const float v = wave_sum4(wr[0].dot(c, f), wr[1].dot(c, f), wr[2].dot(c, f), wr[3].dot(c, f), lane);
            if (lane < 4u && row0 + lane < N) dv[(size_t)a * N + row0 + lane] = v;
        }
    } else {
        for (uint i = a0; i < a1; i++) {
            const uint a = min(list[i], NA - 1u);
            float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            for (uint sb = g; sb < nsb; sb += 8u) {
                Q4kFrag f = q4k_load_frag(aq + (size_t)a * nsb * 256u, as_ + (size_t)a * nsb, sb, l);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    W wr;
                    wr.load(w0 + (size_t)min((uint)r, N - 1u - row0) * rb + (size_t)sb * W::BYTES, l);
                    v[r] += wr.dot(c, f);
                }
            }
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float s = wave_sum(v[r]);
                if (lane == 0 && row0 + r < N) dv[(size_t)a * N + row0 + r] = s;
            }
        }
    }
}
extern "C" __global__ void __launch_bounds__(256)
moe_down_q4k_m(const signed char* aq, const float* as_, const uchar* wd, float* dv, const uint* offsets,
               const uint* list, uint K, uint N, uint NA) {
    moe_down_m_body<W4k>(aq, as_, wd, dv, offsets, list, K, N, NA);
}
// the same over Q5_K rows (an expert's down tensor is often kept a step finer than gate / up)
extern "C" __global__ void __launch_bounds__(256)
moe_down_q5k_m(const signed char* aq, const float* as_, const uchar* wd, float* dv, const uint* offsets,
               const uint* list, uint K, uint N, uint NA) {
    moe_down_m_body<W5k>(aq, as_, wd, dv, offsets, list, K, N, NA);
}
// ... and over Q6_K rows (two steps finer)
extern "C" __global__ void __launch_bounds__(256)
moe_down_q6k_m(const signed char* aq, const float* as_, const uchar* wd, float* dv, const uint* offsets,
               const uint* list, uint K, uint N, uint NA) {
    moe_down_m_body<W6k>(aq, as_, wd, dv, offsets, list, K, N, NA);
}

// ------------------------------------------------------------------ decode: a few tokens, two launches
// With one or a few tokens almost every assignment has its expert to itself, so grouping buys
// nothing and the six launches of the grouped pipeline cost more than the bytes.  Here a workgroup
// is addressed by assignment (gate/up) or by token (down), quantizes the activations it needs into
// LDS itself, and the down projection owns all KSEL slots of its rows, so the router-weighted sum
// happens in the same launch, in slot order.  The arithmetic is that of the grouped integer-dot
// kernels step for step: results are bit-identical.
#define MOE_DEC_GU_K 8192u      // longest row of gate/up the decode form stages (bytes of int8 in LDS)
#define MOE_DEC_DOWN_ACT 32768u // most KSEL * K int8 activations the down launch stages

// All 256 threads: quantize n (a multiple of 256) f32 values into q (int8) and s (one scale per
// 256 values) with quant_q8k's rule (crates/ojas-cpu/src/cpu_math.rs:539-563), the operations of
// the quantize_q8k kernel.  A thread owns 8 consecutive values, 32 lanes side by side a segment.
__device__ __forceinline__ void block_quant_q8k(const float* __restrict__ x, uint n, signed char* q, float* s) {
    for (uint base = threadIdx.x * 8u; base < n; base += 2048u) {
        const float4 a = *(const float4*)(x + base), b = *(const float4*)(x + base + 4u);
        float m = fmaxf(amax4(a), amax4(b));
        m = fmaxf(m, dpp_f32<OJK_DPP_QUAD_XOR1>(m));
        m = fmaxf(m, dpp_f32<OJK_DPP_QUAD_XOR2>(m));
        m = fmaxf(m, dpp_f32<OJK_DPP_ROW_HALF_MIRROR>(m));
        m = fmaxf(m, dpp_f32<OJK_DPP_ROW_MIRROR>(m));
        m = fmaxf(m, __shfl_xor(m, 16, 64));
        const float scale = m > 0.0f ? __fdiv_rn(m, 127.0f) : 1.0f;
        const float inv = __fdiv_rn(1.0f, scale);
        *(uint2*)(q + base) = make_uint2(q8k_pack4(a, inv), q8k_pack4(b, inv));
        if ((threadIdx.x & 31u) == 0) s[base >> 8] = scale;
    }
}

// Where an assignment's expert starts, in bytes from the tensor (or arena) base.  Resident experts
// are indexed (idx[a] * N rows); streamed experts sit wherever the host's cache put them and come
// as one byte offset per assignment (the reference's `_slots` kernels,
// crates/ojas-cuda/src/kernels/moe.rs:133-174).  Offsets are rounded down to 16 bytes and clamped
// to `lim256` * 256, the last offset at which a whole expert still fits.
__device__ __forceinline__ size_t expert_base(const void* sel, uint a, bool slots, uint e_or_lim, size_t expert_bytes) {
    if (slots) {
        const size_t o = (size_t)((const unsigned long*)sel)[a] & ~(size_t)15;
        return min(o, (size_t)e_or_lim * 256u);
    }
    return (size_t)min(((const uint*)sel)[a], e_or_lim - 1u) * expert_bytes;
}

// Block (rb, a): 4 waves x 2 rows of gate and up of assignment a's expert against token a / KSEL.
// ROUTE: the workgroup routes its token itself first — wave 0 runs the router over lg[t], the slot's expert is read
// from LDS, and one workgroup per token writes idx / wgt out for the down launch (sel_g / sel_u are not read).
template <bool SLOTS, bool ROUTE = false>
__device__ __forceinline__ void moe_gu_dec_body(const float* __restrict__ x, const uchar* __restrict__ wg,
                                                const uchar* __restrict__ wu, float* __restrict__ act,
                                                const void* __restrict__ sel_g, const void* __restrict__ sel_u,
                                                uint K, uint N, uint KSEL, uint EG, uint EU,
                                                const float* __restrict__ lg = nullptr, uint* __restrict__ idx_out = nullptr,
                                                float* __restrict__ wgt_out = nullptr) {
    __shared__ __align__(16) signed char xq[MOE_DEC_GU_K];
    __shared__ float xs[MOE_DEC_GU_K / 256u];
    __shared__ uint r_idx[64];
    __shared__ float r_wgt[64];
    uint a = blockIdx.y;
    const uint t = a / KSEL;
    if (ROUTE) {
        if (threadIdx.x < 64u) moe_topk_body(lg + (size_t)t * EG, r_idx, r_wgt, EG, KSEL);
        __syncthreads();
        if (blockIdx.x == 0u && a == t * KSEL && threadIdx.x < KSEL) {
            idx_out[a + threadIdx.x] = r_idx[threadIdx.x];
            wgt_out[a + threadIdx.x] = r_wgt[threadIdx.x];
        }
        sel_g = sel_u = r_idx;
        a -= t * KSEL;              // the slot: index into the token's own table
    }
    const uint lane = threadIdx.x & 63u;
    const uint row0 = min((blockIdx.x * 4u + (threadIdx.x >> 6)) * 2u, N - 1u);   // surplus waves repeat the last row
    const uint nsb = K >> 8, g = lane >> 3, l = lane & 7u, c = l >> 1;
    const size_t rb = (size_t)nsb * Q4K_BYTES;
    const uchar* g0 = wg + expert_base(sel_g, a, SLOTS, EG, (size_t)N * rb) + (size_t)row0 * rb;
    const uchar* u0 = wu + expert_base(sel_u, a, SLOTS, EU, (size_t)N * rb) + (size_t)row0 * rb;
    const bool two = row0 + 1u < N;
    const size_t r1 = two ? rb : 0;
    // the first step's weights are on their way while the activations are quantized
    const size_t o0 = (size_t)min(g, nsb - 1u) * Q4K_BYTES, q0 = o0 + 16u + l * 16u;
    uint4 hg0 = *(const uint4*)(g0 + o0), qg0 = *(const uint4*)(g0 + q0);
    uint4 hg1 = *(const uint4*)(g0 + r1 + o0), qg1 = *(const uint4*)(g0 + r1 + q0);
    uint4 hu0 = *(const uint4*)(u0 + o0), qu0 = *(const uint4*)(u0 + q0);
    uint4 hu1 = *(const uint4*)(u0 + r1 + o0), qu1 = *(const uint4*)(u0 + r1 + q0);
    block_quant_q8k(x + (size_t)t * K, K, xq, xs);
    __syncthreads();
    float vg0 = 0.0f, vg1 = 0.0f, vu0 = 0.0f, vu1 = 0.0f;
    for (uint sb = g; sb < nsb; sb += 8u) {
        const Q4kFrag f = q4k_load_frag(xq, xs, sb, l);
        vg0 += q4k_lane_dot(hg0, qg0, c, f);
        vg1 += q4k_lane_dot(hg1, qg1, c, f);
        vu0 += q4k_lane_dot(hu0, qu0, c, f);
        vu1 += q4k_lane_dot(hu1, qu1, c, f);
        if (sb + 8u < nsb) {
            const size_t o = (size_t)(sb + 8u) * Q4K_BYTES, oq = o + 16u + l * 16u;
            hg0 = *(const uint4*)(g0 + o); qg0 = *(const uint4*)(g0 + oq);
            hg1 = *(const uint4*)(g0 + r1 + o); qg1 = *(const uint4*)(g0 + r1 + oq);
            hu0 = *(const uint4*)(u0 + o); qu0 = *(const uint4*)(u0 + oq);
            hu1 = *(const uint4*)(u0 + r1 + o); qu1 = *(const uint4*)(u0 + r1 + oq);
        }
    }
    vg0 = wave_sum(vg0); vg1 = wave_sum(vg1); vu0 = wave_sum(vu0); vu1 = wave_sum(vu1);
    if (lane == 0) {
        float* o_ = act + (size_t)blockIdx.y * N + row0;
        o_[0] = (vg0 / (1.0f + expf(-vg0))) * vu0;
        if (two) o_[1] = (vg1 / (1.0f + expf(-vg1))) * vu1;
    }
}
extern "C" __global__ void __launch_bounds__(256)
moe_gu_q4k_dec(const float* x, const uchar* wg, const uchar* wu, float* act, const uint* idx, uint K, uint N, uint KSEL,
               uint NA, uint E) {
    moe_gu_dec_body<false>(x, wg, wu, act, idx, idx, K, N, KSEL, E, E);
}
// The decode form with the router inside: moe_gu_q4k_decr(x, wg, wu, act, lg, idx, wgt, K, N, KSEL, NA, E) — lg: the
// router logits [tokens][E]; idx / wgt [tokens][KSEL] are written (softmax, top KSEL, renormalised: moe_topk's
// arithmetic, the same bits) for the down launch that follows.  One launch less per layer and token.
extern "C" __global__ void __launch_bounds__(256)
moe_gu_q4k_decr(const float* x, const uchar* wg, const uchar* wu, float* act, const float* lg, uint* idx, float* wgt,
                uint K, uint N, uint KSEL, uint NA, uint E) {
    moe_gu_dec_body<false, true>(x, wg, wu, act, nullptr, nullptr, K, N, KSEL, E, E, lg, idx, wgt);
}
extern "C" __global__ void __launch_bounds__(256)
moe_gu_q4k_slots(const float* x, const uchar* arena_g, const uchar* arena_u, float* act, const unsigned long* off_g,
                 const unsigned long* off_u, uint K, uint N, uint KSEL, uint NA, uint LIM_G, uint LIM_U) {
    moe_gu_dec_body<true>(x, arena_g, arena_u, act, off_g, off_u, K, N, KSEL, LIM_G, LIM_U);
}

// Block (rb, t): 8 rows of the down projection for every slot of token t, 2 rows per wave.  The
// workgroup quantizes the token's KSEL act vectors into LDS.  An expert's row is short (K / 256 <= 8
// super-blocks, three at the usual 768), so a wave's eight lane groups take (slot, super-block)
// pairs side by side instead of one slot at a time: group sums go through LDS, lane j rebuilds
// slot j's dot with the association of wave_sum, and the slots are added in order,
//     y[t][row] (=, +=) sum_j wgt[t][j] * (Wd_{idx[t][j]} act[t][j])[row].
template <class W, bool SLOTS>
__device__ __forceinline__ void moe_down_dec_body(const float* __restrict__ act, const uchar* __restrict__ wd,
                                                  const void* __restrict__ sel, const float* __restrict__ wgt,
                                                  float* __restrict__ y, uint K, uint N, uint KSEL, uint E, uint ACC) {
    __shared__ __align__(16) signed char aq[MOE_DEC_DOWN_ACT];
    __shared__ float as_[MOE_DEC_DOWN_ACT / 256u];
    __shared__ size_t s_base[64];
    __shared__ __align__(16) float part[4][2][64][8];   // [wave][row][slot][super-block] group sums
    const uint t = blockIdx.y, lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint row0 = min(blockIdx.x * 8u + wave * 2u, N - 1u);   // surplus waves repeat the last row
    const bool two = row0 + 1u < N;
    const uint nsb = K >> 8, G = lane >> 3, l = lane & 7u, c = l >> 1;
    const size_t rb = (size_t)nsb * W::BYTES, r1 = two ? rb : 0;
    const uint U = KSEL * nsb;
    // the first pass's weights are on their way while the activations are quantized
    uint u = min(G, U - 1u), j = u / nsb, sb = u - j * nsb;
    const uchar* w = wd + expert_base(sel, t * KSEL + j, SLOTS, E, (size_t)N * rb) + ((size_t)row0 * nsb + sb) * W::BYTES;
    W w0, w1;
    w0.load(w, l);
    w1.load(w + r1, l);
    if (threadIdx.x < KSEL) s_base[threadIdx.x] = expert_base(sel, t * KSEL + threadIdx.x, SLOTS, E, (size_t)N * rb);
    block_quant_q8k(act + (size_t)t * KSEL * K, KSEL * K, aq, as_);
    __syncthreads();
    for (uint u0 = 0; u0 < U; u0 += 8u) {
        const bool on = u0 + G < U;
        const uint un = min(u0 + 8u + G, U - 1u), jn = un / nsb, sbn = un - jn * nsb;
        const uchar* wn = wd + s_base[jn] + ((size_t)row0 * nsb + sbn) * W::BYTES;
        W n0, n1;
        n0.load(wn, l);
        n1.load(wn + r1, l);
        const Q4kFrag f = q4k_load_frag(aq + (size_t)j * K, as_ + (size_t)j * nsb, sb, l);
        const float v0 = oct_sum(w0.dot(c, f)), v1 = oct_sum(w1.dot(c, f));
        if (on && l == 0) {
            part[wave][0][j][sb] = v0;
            part[wave][1][j][sb] = v1;
        }
        j = jn; sb = sbn; w0 = n0; w1 = n1;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // lane j: slot j's two dots, summed like wave_sum sums the eight groups of a wave
    float d0 = 0.0f, d1 = 0.0f;
    if (lane < KSEL) {
        float s0[8], s1[8];
#pragma unroll
        for (uint k = 0; k < 8; k++) {
            s0[k] = k < nsb ? part[wave][0][lane][k] : 0.0f;
            s1[k] = k < nsb ? part[wave][1][lane][k] : 0.0f;
        }
        d0 = ((s0[0] + s0[1]) + (s0[2] + s0[3])) + ((s0[4] + s0[5]) + (s0[6] + s0[7]));
        d1 = ((s1[0] + s1[1]) + (s1[2] + s1[3])) + ((s1[4] + s1[5]) + (s1[6] + s1[7]));
    }
    float acc0 = 0.0f, acc1 = 0.0f;
    if (ACC) {
        acc0 = y[(size_t)t * N + row0];
        acc1 = y[(size_t)t * N + row0 + (two ? 1u : 0u)];
    }
    for (uint k = 0; k < KSEL; k++) {
        const float wk = wgt[(size_t)t * KSEL + k];
        acc0 += wk * __int_as_float(__builtin_amdgcn_readlane(__float_as_int(d0), k));
        acc1 += wk * __int_as_float(__builtin_amdgcn_readlane(__float_as_int(d1), k));
    }
    if (lane == 0) {
        y[(size_t)t * N + row0] = acc0;
        if (two) y[(size_t)t * N + row0 + 1u] = acc1;
    }
}
extern "C" __global__ void __launch_bounds__(256)
moe_down_q4k_dec(const float* act, const uchar* wd, const uint* idx, const float* wgt, float* y, uint K, uint N,
                 uint KSEL, uint E, uint ACC) {
    moe_down_dec_body<W4k, false>(act, wd, idx, wgt, y, K, N, KSEL, E, ACC);
}
extern "C" __global__ void __launch_bounds__(256)
moe_down_q4k_slots(const float* act, const uchar* arena, const unsigned long* off_d, const float* wgt, float* y, uint K,
                   uint N, uint KSEL, uint LIM, uint ACC) {
    moe_down_dec_body<W4k, true>(act, arena, off_d, wgt, y, K, N, KSEL, LIM, ACC);
}
extern "C" __global__ void __launch_bounds__(256)
moe_down_q5k_dec(const float* act, const uchar* wd, const uint* idx, const float* wgt, float* y, uint K, uint N,
                 uint KSEL, uint E, uint ACC) {
    moe_down_dec_body<W5k, false>(act, wd, idx, wgt, y, K, N, KSEL, E, ACC);
}
extern "C" __global__ void __launch_bounds__(256)
moe_down_q6k_dec(const float* act, const uchar* wd, const uint* idx, const float* wgt, float* y, uint K, uint N,
                 uint KSEL, uint E, uint ACC) {
    moe_down_dec_body<W6k, false>(act, wd, idx, wgt, y, K, N, KSEL, E, ACC);
}

// ------------------------------------------------------------------ the quantizer and the grouping in one launch
//   moe_quant_group(x, xq, xs, idx, counts, offsets, list, K, T, NA, E)   grid [T + 1,1,1]: block t quantizes token t
//       (quant_q8k's rule, the operations of quantize_q8k), the last block sorts the assignments by expert (moe_group).
// Neither depends on the other; both are a few microseconds of launch and little else.
extern "C" __global__ void __launch_bounds__(256)
moe_quant_group(const float* __restrict__ x, signed char* __restrict__ xq, float* __restrict__ xs, const uint* __restrict__ idx,
                uint* __restrict__ counts, uint* __restrict__ offsets, uint* __restrict__ list, uint K, uint T, uint NA, uint E) {
    __shared__ uint cnt[1024];
    __shared__ uint off[1025];
    if (blockIdx.x >= T) {
        moe_group_body(idx, counts, offsets, list, NA, E, cnt, off);
        return;
    }
    const size_t t = blockIdx.x;
    block_quant_q8k(x + t * K, K, xq + t * K, xs + t * (K >> 8));
}

// ------------------------------------------------------------------ Q8_0 experts, f32 activations
//   moe_gu_q80(x, wg, wu, act, idx, K, N)              grid [ceil(N/8), KSEL, tokens], block 256
//   moe_down_q80(act, wd, y, idx, wgt, K, N, KSEL)     grid [1 .. ceil(N/4), tokens, 1], block 256 (rows grid-stride,
//                                                      4 per workgroup and step: the reference's ceil(N/32) is a valid grid)
// The reference's expert kernels by their own names and arguments
// (crates/ojas-cuda/src/kernels/moe.rs:75-125): act[j][n] = silu(gate_e . x) * (up_e . x) for the expert
// e = idx[j] of slot j, and y[n] += sum_j wgt[j] * (down_e . act[j]) — the down launch accumulates onto y.  Q8_0 rows meet f32 activations, as dot_q80 does
// (crates/ojas-cpu/src/cpu_math.rs:971-981).  The third (second) grid dimension walks tokens: token t
// reads x + t K, idx + t KSEL, wgt + t KSEL and writes act + t KSEL N, y + t N; a one-token caller
// leaves it at 1.  Four lanes share a 34-byte block, a wave walks 16 blocks per step.  The trailing E is
// not part of the reference's argument list: the dispatcher derives it from the extent of the expert
// tensors, and a slot whose index is E or more contributes zeros rather than reading past them.
__device__ __forceinline__ float q80f_block_part(const uchar* blk, uint p, float4 x0, float4 x1) {
    const u32x2_a2 q = *(const u32x2_a2*)(blk + 2u + p * 8u);
    float a = (float)(signed char)(q.x) * x0.x;
    a = fmaf((float)(signed char)(q.x >> 8), x0.y, a);
    a = fmaf((float)(signed char)(q.x >> 16), x0.z, a);
    a = fmaf((float)((int)q.x >> 24), x0.w, a);
    a = fmaf((float)(signed char)(q.y), x1.x, a);
    a = fmaf((float)(signed char)(q.y >> 8), x1.y, a);
    a = fmaf((float)(signed char)(q.y >> 16), x1.z, a);
    a = fmaf((float)((int)q.y >> 24), x1.w, a);
    return f16_bits_to_f32(*(const ushort*)blk) * a;
}

// gate/up rows of one expert (eg, eu: its first rows) against token row xt; nb = 0 skips the products
__device__ __forceinline__ void moe_gu_q80_body(const float* __restrict__ xt, const uchar* __restrict__ eg,
                                                const uchar* __restrict__ eu, float* __restrict__ act_row,
                                                uint K, uint N, uint nb) {
    const uint lane = threadIdx.x & 63u, g = lane >> 2, p = lane & 3u;
    const uint row0 = (blockIdx.x * 4u + (threadIdx.x >> 6)) * 2u;
    if (row0 >= N) return;
    const size_t rb = (size_t)(K >> 5) * Q80_BYTES;
    float ag[2] = {0.0f, 0.0f}, au[2] = {0.0f, 0.0f};
    for (uint b = g; b < nb; b += 16u) {
        const float4* xp = (const float4*)(xt + (size_t)b * 32u + p * 8u);
        const float4 x0 = xp[0], x1 = xp[1];
#pragma unroll
        for (int r = 0; r < 2; r++) {
            const size_t off = (size_t)min(row0 + (uint)r, N - 1u) * rb + (size_t)b * Q80_BYTES;
            ag[r] += q80f_block_part(eg + off, p, x0, x1);
            au[r] += q80f_block_part(eu + off, p, x0, x1);
        }
    }
#pragma unroll
    for (int r = 0; r < 2; r++) {
        const float gs = wave_sum(ag[r]), us = wave_sum(au[r]);
        if (lane == 0 && row0 + r < N) act_row[row0 + r] = (gs / (1.0f + expf(-gs))) * us;
    }
}

// four down rows of one expert (ed: its first row) against one activation row
__device__ __forceinline__ void moe_down_q80_part(const float* __restrict__ xr, const uchar* __restrict__ ed,
                                                  uint K, uint N, uint row0, float wj, float (&res)[4]) {
    const uint lane = threadIdx.x & 63u, g = lane >> 2, p = lane & 3u;
    const uint nb = K >> 5;
    const size_t rb = (size_t)nb * Q80_BYTES;
    float a[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (uint b = g; b < nb; b += 16u) {
        const float4* xp = (const float4*)(xr + (size_t)b * 32u + p * 8u);
        const float4 x0 = xp[0], x1 = xp[1];
#pragma unroll
        for (int r = 0; r < 4; r++)
            a[r] += q80f_block_part(ed + (size_t)min(row0 + (uint)r, N - 1u) * rb + (size_t)b * Q80_BYTES, p, x0, x1);
    }
#pragma unroll
    for (int r = 0; r < 4; r++) res[r] += wj * wave_sum(a[r]);
}

extern "C" __global__ void __launch_bounds__(256)
moe_gu_q80(const float* __restrict__ x, const uchar* __restrict__ wg, const uchar* __restrict__ wu,
           float* __restrict__ act, const uint* __restrict__ idx, uint K, uint N, uint E) {
    const uint j = blockIdx.y, t = blockIdx.z, ksel = gridDim.y;
    const uint e = idx[t * ksel + j];
    const size_t eb = (size_t)(e < E ? e : 0u) * N * ((size_t)(K >> 5) * Q80_BYTES);
    moe_gu_q80_body(x + (size_t)t * K, wg + eb, wu + eb, act + ((size_t)t * ksel + j) * N, K, N, e < E ? K >> 5 : 0u);
}

// The down launches: a workgroup owns four rows at a time (rows grid-stride over the workgroups), its four
// waves take the slots j = wave, wave + 4, ... and meet in LDS, where the partial sums are added in wave order
// onto y — an expert row is short (a few hundred to a few thousand weights), so the slots are the parallelism
// that fills the chip at one token.
__device__ __forceinline__ void moe_down_finish(float (&res)[4], float* __restrict__ yt, uint N, uint row0) {
    __shared__ float part[4][4];
    const uint lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < 4; r++) part[wave][r] = res[r];
    }
    __syncthreads();
    if (threadIdx.x < 4u && row0 + threadIdx.x < N)
        yt[row0 + threadIdx.x] += ((part[0][threadIdx.x] + part[1][threadIdx.x]) + part[2][threadIdx.x]) + part[3][threadIdx.x];
    __syncthreads();
}

extern "C" __global__ void __launch_bounds__(256)
moe_down_q80(const float* __restrict__ act, const uchar* __restrict__ wd, float* __restrict__ y,
             const uint* __restrict__ idx, const float* __restrict__ wgt, uint K, uint N, uint KSEL, uint E) {
    const uint t = blockIdx.y, wave = threadIdx.x >> 6;
    const size_t eb = (size_t)N * ((size_t)(K >> 5) * Q80_BYTES);
    for (uint row0 = blockIdx.x * 4u; row0 < N; row0 += gridDim.x * 4u) {
        float res[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (uint j = wave; j < KSEL; j += 4u) {
            const uint e = idx[t * KSEL + j];
            if (e >= E) continue;
            moe_down_q80_part(act + ((size_t)t * KSEL + j) * K, wd + (size_t)e * eb, K, N, row0, wgt[t * KSEL + j], res);
        }
        moe_down_finish(res, y + (size_t)t * N, N, row0);
    }
}

// Streamed Q8_0 experts (crates/ojas-cuda/src/kernels/moe.rs:133-174): the experts of a layer sit at whatever
// slots of a cache arena were free, and the host passes one u32 byte offset per selected expert in place of
// the index.   moe_gu_q80_slots(x, arena_g, arena_u, act, off_g, off_u, K, N)   grid [ceil(N/8), KSEL, tokens]
//              moe_down_q80_slots(act, arena, y, off_d, wgt, K, N, KSEL)          grid [1 .. ceil(N/4), tokens, 1]
// The trailing LIM constants are appended by the dispatcher — the last offset at which a whole expert still
// fits its arena — and an offset is rounded down to the blocks' two-byte alignment and clamped to LIM, so a bad
// table reads a wrong expert, never past the arena.
extern "C" __global__ void __launch_bounds__(256)
moe_gu_q80_slots(const float* __restrict__ x, const uchar* __restrict__ arena_g, const uchar* __restrict__ arena_u,
                 float* __restrict__ act, const uint* __restrict__ off_g, const uint* __restrict__ off_u,
                 uint K, uint N, uint LIM_G, uint LIM_U) {
    const uint j = blockIdx.y, t = blockIdx.z, ksel = gridDim.y;
    const uint og = min(off_g[t * ksel + j] & ~1u, LIM_G), ou = min(off_u[t * ksel + j] & ~1u, LIM_U);
    moe_gu_q80_body(x + (size_t)t * K, arena_g + og, arena_u + ou, act + ((size_t)t * ksel + j) * N, K, N, K >> 5);
}

extern "C" __global__ void __launch_bounds__(256)
moe_down_q80_slots(const float* __restrict__ act, const uchar* __restrict__ arena, float* __restrict__ y,
                   const uint* __restrict__ off_d, const float* __restrict__ wgt, uint K, uint N, uint KSEL, uint LIM) {
    const uint t = blockIdx.y, wave = threadIdx.x >> 6;
    for (uint row0 = blockIdx.x * 4u; row0 < N; row0 += gridDim.x * 4u) {
        float res[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (uint j = wave; j < KSEL; j += 4u)
            moe_down_q80_part(act + ((size_t)t * KSEL + j) * K, arena + min(off_d[t * KSEL + j] & ~1u, LIM), K, N, row0,
                              wgt[t * KSEL + j], res);
        moe_down_finish(res, y + (size_t)t * N, N, row0);
    }
}

// ------------------------------------------------------------------ grouped products on the matrix cores
// A workgroup owns 16 rows of expert e and walks the expert's assignments 16 at a time.  Per 32-weight
// sub-block one v_mfma_i32_16x16x32_i8 multiplies the tile of quantized activations (A: lane
// (m, kg) = (lane % 16, lane / 16) holds bytes 8 kg .. 8 kg + 7 of token m) with the sub-block's
// 4-bit codes as bytes (B: lane (n, kg) holds the same bytes of row n); D register v of lane
// (n, kg) is the integer dot of token 4 kg + v with row n.  A second MFMA against a tile of ones
// gives every lane the activations' sub-block sums in the same layout, so the scale algebra
//     sum_sb sx[t][sb] * ( d * sum_j sc_j * idot_j  -  dmin * sum_j m_j * bsum_j )
// needs no cross-lane traffic: per MFMA result register one integer multiply-add with a
// lane-constant 6-bit scale (the sums over j are exact in int32: |.| < 2^25), and per super-block
// two converts and three FMAs, the form of dot_q4k itself (crates/ojas-cpu/src/cpu_math.rs:609-635).  A token's result does not
// depend on which other tokens share its tile.
typedef int int4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ long pack2(uint lo, uint hi) { return (long)(((unsigned long)hi << 32) | lo); }

// acc[w][v] += sx[v] * sum_j (a_j * idot_j[v] - b_j * bsum_j[v]) for one super-block of NW weight
// tensors sharing the activations.  `xsb` points at the lane's 8 bytes of sub-block 0 (sub-block j
// 32 bytes further); `wblk[w]` at the lane's row inside a wave-private LDS copy of the 16 x 144-byte
// tile.
template <int NW>
__device__ __forceinline__ void mm_superblock(const signed char* xsb, const uchar* const (&wblk)[NW], uint kg,
                                              const float (&sx)[4], float (&acc)[NW][4]) {
    // integer partial sums are exact, so sum_j sc_j * idot_j and sum_j m_j * bsum_j are formed in
    // int32 (one v_mad_i32_i24 per MFMA result register) and converted once per super-block
    int isum[NW][4], msum[NW][4];
    float d[NW], dmin[NW];
    uint s0[NW], s1[NW], s2[NW];
#pragma unroll
    for (int w = 0; w < NW; w++) {
        const uint4 hdr = *(const uint4*)wblk[w];
        d[w] = f16_bits_to_f32(hdr.x & 0xFFFFu);
        dmin[w] = f16_bits_to_f32(hdr.x >> 16);
        s0[w] = hdr.y; s1[w] = hdr.z; s2[w] = hdr.w;
#pragma unroll
        for (int v = 0; v < 4; v++) { isum[w][v] = 0; msum[w][v] = 0; }
    }
    const long ones = 0x0101010101010101L;
    const int4v zero = {0, 0, 0, 0};
    // (kept rolled: unrolled, the compiler holds every scale and code of the super-block at once,
    // occupancy drops, and the kernel measured slower)
#pragma unroll 1
    for (uint c = 0; c < 4u; c++) {
        const uint2 x0 = *(const uint2*)(xsb + c * 64u), x1 = *(const uint2*)(xsb + c * 64u + 32u);
        const long A0 = pack2(x0.x, x0.y), A1 = pack2(x1.x, x1.y);
        const int4v b0 = __builtin_amdgcn_mfma_i32_16x16x32_i8(A0, ones, zero, 0, 0, 0);
        const int4v b1 = __builtin_amdgcn_mfma_i32_16x16x32_i8(A1, ones, zero, 0, 0, 0);
#pragma unroll
        for (int w = 0; w < NW; w++) {
            uint sc, mn;
            q4k_scale_min_pair(s0[w], s1[w], s2[w], c, sc, mn);
            const int sc_lo = (int)(sc & 0xFFu), sc_hi = (int)(sc >> 8), m_lo = (int)(mn & 0xFFu), m_hi = (int)(mn >> 8);
            const uint2 q = *(const uint2*)(wblk[w] + 16u + c * 32u + 8u * kg);
            const int4v dl = __builtin_amdgcn_mfma_i32_16x16x32_i8(A0, pack2(q.x & 0x0F0F0F0Fu, q.y & 0x0F0F0F0Fu), zero, 0, 0, 0);
            const int4v dh = __builtin_amdgcn_mfma_i32_16x16x32_i8(A1, pack2((q.x >> 4) & 0x0F0F0F0Fu, (q.y >> 4) & 0x0F0F0F0Fu), zero, 0, 0, 0);
#pragma unroll
            for (int v = 0; v < 4; v++) {
                isum[w][v] += __mul24(sc_lo, dl[v]) + __mul24(sc_hi, dh[v]);
                msum[w][v] += __mul24(m_lo, b0[v]) + __mul24(m_hi, b1[v]);
            }
        }
    }
#pragma unroll
    for (int w = 0; w < NW; w++)
#pragma unroll
        for (int v = 0; v < 4; v++) acc[w][v] += sx[v] * (d[w] * (float)isum[w][v] - dmin[w] * (float)msum[w][v]);
}

// Copy the super-block `sb` of 16 consecutive rows (144 bytes each, `rb` apart, rows past `nrows`
// clamped) into the wave's LDS tile with 16-byte pieces, 64 lanes side by side: the loads are
// contiguous per row instead of 8 bytes per lane and row.
__device__ __forceinline__ void mm_stage_tile(const uchar* w_row0, size_t rb, uint nrows, uint sb, uchar* tile, uint lane) {
#pragma unroll
    for (int i = 0; i < 3; i++) {
        const uint p = lane + 64u * i;
        if (p < 144u) {
            const uint r = p / 9u, c = p - r * 9u;
            *(uint4*)(tile + p * 16u) = *(const uint4*)(w_row0 + (size_t)min(r, nrows - 1u) * rb + (size_t)sb * Q4K_BYTES + c * 16u);
        }
    }
}

// Workgroup = one 16-row tile of expert e; its four waves split the super-blocks of K between
// them (wave w takes w, w + 4, ...) and their partial sums meet in LDS, added in wave order.
template <int NW>
__device__ __forceinline__ void mm_reduce(float (&acc)[NW][4], float* red, uint wave, uint lane) {
    // red: [3 waves][NW * 4][64 lanes]
    if (wave > 0) {
#pragma unroll
        for (int w = 0; w < NW; w++)
#pragma unroll
            for (int v = 0; v < 4; v++) red[((wave - 1u) * (NW * 4) + w * 4 + v) * 64u + lane] = acc[w][v];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
        for (int k = 0; k < 3; k++)
#pragma unroll
            for (int w = 0; w < NW; w++)
#pragma unroll
                for (int v = 0; v < 4; v++) acc[w][v] += red[(k * (NW * 4) + w * 4 + v) * 64u + lane];
    }
    __syncthreads();
}

// (four waves per SIMD: latency of the dependent list -> activation -> weight loads is hidden by occupancy)
extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 8)))
moe_gu_q4k_mm(const signed char* __restrict__ xq, const float* __restrict__ xs, const uchar* __restrict__ wg,
              const uchar* __restrict__ wu, float* __restrict__ act, const uint* __restrict__ offsets,
              const uint* __restrict__ list, uint K, uint N, uint KSEL, uint NA) {
    __shared__ float red[3 * 8 * 64];
    __shared__ __attribute__((aligned(16))) uchar tiles[4][2][16 * Q4K_BYTES];
    const uint e = blockIdx.y;
    const uint a0 = min(offsets[e], NA), a1 = min(offsets[e + 1], NA);
    if (a0 >= a1) return;
    const uint lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, n = lane & 15u, kg = lane >> 4;
    const uint row0 = blockIdx.x * 16u;
    const uint nsb = K >> 8;
    const size_t rb = (size_t)nsb * Q4K_BYTES;
    const uchar* gw = wg + ((size_t)e * N + row0) * rb;
    const uchar* uw = wu + ((size_t)e * N + row0) * rb;
    const uint nrows = min(16u, N - row0);
    for (uint tt = a0; tt < a1; tt += 16u) {
        // activations: lane's token for the A operand, and the four tokens of its D registers
        const uint ta = min(list[min(tt + n, a1 - 1u)], NA - 1u) / KSEL;
        const signed char* xrow = xq + (size_t)ta * K + 8u * kg;
        uint av[4], tv[4];
#pragma unroll
        for (int v = 0; v < 4; v++) {
            av[v] = min(list[min(tt + 4u * kg + v, a1 - 1u)], NA - 1u);
            tv[v] = av[v] / KSEL;
        }
        float acc[2][4];
#pragma unroll
        for (int w = 0; w < 2; w++)
#pragma unroll
            for (int v = 0; v < 4; v++) acc[w][v] = 0.0f;
#pragma unroll 1
        for (uint sb = wave; sb < nsb; sb += 4u) {
            float sx[4];
#pragma unroll
            for (int v = 0; v < 4; v++) sx[v] = xs[(size_t)tv[v] * nsb + sb];
            mm_stage_tile(gw, rb, nrows, sb, tiles[wave][0], lane);
            mm_stage_tile(uw, rb, nrows, sb, tiles[wave][1], lane);
            const uchar* const wb[2] = {tiles[wave][0] + n * Q4K_BYTES, tiles[wave][1] + n * Q4K_BYTES};
            mm_superblock<2>(xrow + sb * 256u, wb, kg, sx, acc);
        }
        mm_reduce<2>(acc, red, wave, lane);
        if (wave == 0 && row0 + n < N) {
#pragma unroll
            for (int v = 0; v < 4; v++)
                if (tt + 4u * kg + v < a1) {
                    const float g = acc[0][v];
                    act[(size_t)av[v] * N + row0 + n] = (g / (1.0f + expf(-g))) * acc[1][v];
                }
        }
    }
}

extern "C" __global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 8)))
moe_down_q4k_mm(const signed char* __restrict__ aq, const float* __restrict__ as_, const uchar* __restrict__ wd,
                float* __restrict__ dv, const uint* __restrict__ offsets, const uint* __restrict__ list,
                uint K, uint N, uint NA) {
    __shared__ float red[3 * 4 * 64];
    __shared__ __attribute__((aligned(16))) uchar tiles[4][16 * Q4K_BYTES];
    const uint e = blockIdx.y;
    const uint a0 = min(offsets[e], NA), a1 = min(offsets[e + 1], NA);
    if (a0 >= a1) return;
    const uint lane = threadIdx.x & 63u, wave = threadIdx.x >> 6, n = lane & 15u, kg = lane >> 4;
    const uint row0 = blockIdx.x * 16u;
    const uint nsb = K >> 8;
    const size_t rb = (size_t)nsb * Q4K_BYTES;
    const uchar* dw = wd + ((size_t)e * N + row0) * rb;
    const uint nrows = min(16u, N - row0);
    for (uint tt = a0; tt < a1; tt += 16u) {
        const uint aa = min(list[min(tt + n, a1 - 1u)], NA - 1u);
        const signed char* xrow = aq + (size_t)aa * K + 8u * kg;
        uint av[4];
#pragma unroll
        for (int v = 0; v < 4; v++) av[v] = min(list[min(tt + 4u * kg + v, a1 - 1u)], NA - 1u);
        float acc[1][4] = {{0.0f, 0.0f, 0.0f, 0.0f}};
#pragma unroll 1
        for (uint sb = wave; sb < nsb; sb += 4u) {
            float sx[4];
#pragma unroll
            for (int v = 0; v < 4; v++) sx[v] = as_[(size_t)av[v] * nsb + sb];
            mm_stage_tile(dw, rb, nrows, sb, tiles[wave], lane);
            const uchar* const wb[1] = {tiles[wave] + n * Q4K_BYTES};
            mm_superblock<1>(xrow + sb * 256u, wb, kg, sx, acc);
        }
        mm_reduce<1>(acc, red, wave, lane);
        if (wave == 0 && row0 + n < N) {
#pragma unroll
            for (int v = 0; v < 4; v++)
                if (tt + 4u * kg + v < a1) dv[(size_t)av[v] * N + row0 + n] = acc[0][v];
        }
    }
}

// ------------------------------------------------------------------ grouped products, a wave per row tile
//   moe_gu_q4k_mt / moe_down_q4k_mt (the arguments of the _m entries)   grid [RG, E, 1], block 512,
//                                                                       16 (K + 32) + 5 K / 4 + 320 <= 81920
// With many small experts (128 x 768 x 2048) the _mm form spends its time around the products: a
// workgroup per 16-row tile and expert (16384 of them for the down matrices, three super-blocks
// each), activations fetched from global memory per super-block, partial sums of four waves
// through LDS.  Here RG workgroups share an expert: each stages the expert's next 16 assignments
// once (token rows gathered through the list into LDS, scales, sums split into int8 parts; rows
// past the count are one block of zeros), then every wave walks whole row tiles, all of K, with
// the dense entries' super-block routine (10 MFMAs instead of 24 per super-block and tensor
// pair) and writes its own outputs; no partial sums meet.  Tile i of the expert belongs to
// workgroup i % RG, wave (i / RG) % 8.  Super-blocks are added in order.
#define MT_LDS 81920u
// A pass stages 16 P assignments; P = 2 where 32 token rows fit (32 (K + 32) + 5 K / 2 + 384 <= 81920): an expert with
// 17 .. 32 assignments then has its rows read and unpacked once instead of twice (at 256 tokens over 128 experts with
// 8 slots each, 16 per expert on average, that is every other expert).
template <bool GU, int P>
__device__ __forceinline__ void moe_mt_body(const signed char* __restrict__ xq, const float* __restrict__ xs,
                                            const uchar* __restrict__ w0, const uchar* __restrict__ w1, float* __restrict__ out,
                                            const uint* __restrict__ offsets, const uint* __restrict__ list,
                                            uint K, uint N, uint KSEL, uint NA, uchar* lds) {
    constexpr uint TP = 16u * P;
    constexpr int NT = GU ? 2 : 1;
    const uint e = blockIdx.y;
    const uint a0 = min(offsets[e], NA), a1 = min(offsets[e + 1], NA);
    if (a0 >= a1) return;
    const uint tid = threadIdx.x, lane = tid & 63u, nt = blockDim.x;
    const uint wave = (uint)__builtin_amdgcn_readfirstlane((int)(tid >> 6)), nw = nt >> 6;
    const uint nsb = K >> 8, S = K + 32u, per_row = K >> 4;
    const uint o_lsx = TP * S, o_lbq = o_lsx + nsb * TP * 4u, o_zero = o_lbq + nsb * TP * 16u, o_av = o_zero + 256u;
    float* lsx = (float*)(lds + o_lsx);            // [sb][TP] token scales
    uchar* lbq = lds + o_lbq;                      // [sb][TP][16]: lo_0..7, hi_0..7 of the bsums
    uint* lav = (uint*)(lds + o_av);               // [TP] the pass's assignments
    if (tid < 64u) ((uint*)(lds + o_zero))[tid] = 0u;
    const uint n = lane & 15u, kg = lane >> 4;
    const size_t rb = (size_t)nsb * Q4K_BYTES;
    const uint tiles = (N + 15u) >> 4;
    for (uint tt = a0; tt < a1; tt += TP) {
        const uint cnt = min(TP, a1 - tt);
        __syncthreads();                           // the previous pass is done with the staged tokens
        if (tid < TP) lav[tid] = min(list[min(tt + tid, a1 - 1u)], NA - 1u);
        __syncthreads();
        // token rows 0 .. cnt - 1, eight loads in flight per thread
        const uint total = cnt * per_row;
        for (uint i0 = tid; i0 < total; i0 += 8u * nt) {
            uint4 v[8];
            uint dst[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const uint i = i0 + (uint)u * nt, t = min(i / per_row, TP - 1u), o = (i - (i / per_row) * per_row) << 4;
                const uint src = GU ? lav[t] / KSEL : lav[t];
                v[u] = make_uint4(0u, 0u, 0u, 0u);
                dst[u] = t * S + o;
                if (i < total) v[u] = *(const uint4*)(xq + (size_t)src * K + o);
            }
#pragma unroll
            for (int u = 0; u < 8; u++)
                if (i0 + (uint)u * nt < total) *(uint4*)(lds + dst[u]) = v[u];
        }
        for (uint i = tid; i < nsb * TP; i += nt) {
            const uint sb = i / TP, t = i - sb * TP;
            const uint src = GU ? lav[t] / KSEL : lav[t];
            lsx[i] = t < cnt ? xs[(size_t)src * nsb + sb] : 0.0f;
        }
        __syncthreads();
        for (uint i = tid; i < nsb * TP * 8u; i += nt) {
            const uint jj = i & 7u, t = (i >> 3) % TP, sb = (i >> 3) / TP;
            int bs = 0;
            if (t < cnt) {
                const uint4* px = (const uint4*)(lds + (size_t)t * S + sb * 256u + jj * 32u);
                const uint4 a = px[0], b = px[1];
                bs = dot4_i8(a.x, 0x01010101u, 0);
                bs = dot4_i8(a.y, 0x01010101u, bs); bs = dot4_i8(a.z, 0x01010101u, bs); bs = dot4_i8(a.w, 0x01010101u, bs);
                bs = dot4_i8(b.x, 0x01010101u, bs); bs = dot4_i8(b.y, 0x01010101u, bs);
                bs = dot4_i8(b.z, 0x01010101u, bs); bs = dot4_i8(b.w, 0x01010101u, bs);
            }
            uchar* o = lbq + ((size_t)sb * TP + t) * 16u;
            o[jj] = (uchar)(bs & 63);
            o[8u + jj] = (uchar)(bs >> 6);
        }
        __syncthreads();
        const uint np = (cnt + 15u) >> 4;          // token tiles of 16 this pass holds
        const uchar* xa[P];
        uint xstep[P];
#pragma unroll
        for (int p = 0; p < P; p++) {
            const bool on = n + 16u * p < cnt;
            xa[p] = on ? lds + (size_t)(n + 16u * p) * S + 8u * kg : lds + o_zero + 8u * kg;
            xstep[p] = on ? 256u : 0u;
        }
        // This wave's tiles as one stream of (tile, super-block) steps, the blocks of three steps on their
        // way: a wave that loads a step only when it starts the one before it walks a chain of memory
        // latencies (32 of them per pass at 768 x 2048) and the launch is bound by that chain.
        const uint first = wave * gridDim.x + blockIdx.x, stride = nw * gridDim.x;
        const uint my_tiles = first < tiles ? (tiles - first + stride - 1u) / stride : 0u;
        const uint steps = my_tiles * nsb;
        uint i_u = 0u, i_sb = 0u, i_tile = first;
        auto next_step = [&](GqW (&blk)[NT]) {   // loads past the last step repeat it
            const size_t off = ((size_t)e * N + min(i_tile * 16u + n, N - 1u)) * rb + (size_t)i_sb * Q4K_BYTES;
            blk[0] = gq_load(w0 + off, kg);
            if (GU) blk[NT - 1] = gq_load(w1 + off, kg);
            if (i_u + 1u < steps) {
                i_u++;
                if (++i_sb == nsb) {
                    i_sb = 0u;
                    i_tile += stride;
                }
            }
        };
        if (steps == 0u) continue;
        GqW c0[NT], c1[NT], c2[NT];
        next_step(c0);
        next_step(c1);
        next_step(c2);
        float acc[NT][P][4];
#pragma unroll
        for (int w = 0; w < NT; w++)
#pragma unroll
            for (int p = 0; p < P; p++)
#pragma unroll
                for (int v = 0; v < 4; v++) acc[w][p][v] = 0.0f;
        uint c_sb = 0u, c_tile = first;
        for (uint u = 0; u < steps; u++) {
            GqW c3[NT];
            next_step(c3);
#pragma unroll
            for (int w = 0; w < NT; w++)
#pragma unroll
                for (int p = 0; p < P; p++)
                    if ((uint)p < np)
                        gq_superblock(c0[w], xa[p] + c_sb * xstep[p], lbq + ((size_t)c_sb * TP + 16u * p + n) * 16u,
                                      lsx + c_sb * TP + 16u * p, kg, acc[w][p]);
#pragma unroll
            for (int w = 0; w < NT; w++) {
                c0[w] = c1[w];
                c1[w] = c2[w];
                c2[w] = c3[w];
            }
            if (++c_sb == nsb) {
                // D register v of lane (n, kg): assignment 16 p + 4 kg + v of the pass, row n of the tile
                if (c_tile * 16u + n < N) {
#pragma unroll
                    for (int p = 0; p < P; p++)
#pragma unroll
                        for (int v = 0; v < 4; v++) {
                            const uint t = 16u * p + 4u * kg + (uint)v;
                            if (t < cnt) {
                                float* o = out + (size_t)lav[t] * N + c_tile * 16u + n;
                                if (GU) {
                                    const float g = acc[0][p][v];
                                    *o = (g / (1.0f + expf(-g))) * acc[NT - 1][p][v];
                                } else {
                                    *o = acc[0][p][v];
                                }
                            }
                        }
                }
#pragma unroll
                for (int w = 0; w < NT; w++)
#pragma unroll
                    for (int p = 0; p < P; p++)
#pragma unroll
                        for (int v = 0; v < 4; v++) acc[w][p][v] = 0.0f;
                c_sb = 0u;
                c_tile += stride;
            }
        }
    }
}

extern "C" __global__ void __launch_bounds__(512)
moe_gu_q4k_mt(const signed char* __restrict__ xq, const float* __restrict__ xs, const uchar* __restrict__ wg,
              const uchar* __restrict__ wu, float* __restrict__ act, const uint* __restrict__ offsets,
              const uint* __restrict__ list, uint K, uint N, uint KSEL, uint NA) {
    __shared__ __attribute__((aligned(16))) uchar lds_mt[MT_LDS];
    if (32u * (K + 32u) + 5u * (K >> 1) + 384u <= MT_LDS) moe_mt_body<true, 2>(xq, xs, wg, wu, act, offsets, list, K, N, KSEL, NA, lds_mt);
    else moe_mt_body<true, 1>(xq, xs, wg, wu, act, offsets, list, K, N, KSEL, NA, lds_mt);
}

extern "C" __global__ void __launch_bounds__(512)
moe_down_q4k_mt(const signed char* __restrict__ aq, const float* __restrict__ as_, const uchar* __restrict__ wd,
                float* __restrict__ dv, const uint* __restrict__ offsets, const uint* __restrict__ list,
                uint K, uint N, uint NA) {
    __shared__ __attribute__((aligned(16))) uchar lds_mt[MT_LDS];
    if (32u * (K + 32u) + 5u * (K >> 1) + 384u <= MT_LDS) moe_mt_body<false, 2>(aq, as_, wd, wd, dv, offsets, list, K, N, 1u, NA, lds_mt);
    else moe_mt_body<false, 1>(aq, as_, wd, wd, dv, offsets, list, K, N, 1u, NA, lds_mt);
}

// ------------------------------------------------------------------ combine
// y[t][i] (=, +=) sum_j wgt[t][j] * dv[t*KSEL + j][i], slots in order.
extern "C" __global__ void __launch_bounds__(256)
moe_combine(const float* __restrict__ dv, const float* __restrict__ wgt, float* __restrict__ y,
            uint T, uint KSEL, uint D, uint ACC) {
    const size_t i = (size_t)blockIdx.x * 256u + threadIdx.x;
    if (i >= (size_t)T * D) return;
    const uint t = (uint)(i / D), col = (uint)(i % D);
    float acc = ACC ? y[i] : 0.0f;
    // (eight slots' loads in flight before the first is added — slot order kept; past the last slot they repeat it)
    for (uint j0 = 0; j0 < KSEL; j0 += 8u) {
        float w[8], d[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const size_t a = (size_t)t * KSEL + min(j0 + (uint)u, KSEL - 1u);
            w[u] = wgt[a];
            d[u] = dv[a * D + col];
        }
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (j0 + (uint)u < KSEL) acc += w[u] * d[u];
    }
    y[i] = acc;
}

// ------------------------------------------------------------------ K-quant experts on f32 activations
// The reference's expert kernels for raw K-quant rows under their own names (the expert table,
// crates/ojas-core/src/quant_src.rs:168-193; bodies crates/ojas-metal/src/kernels/moe.rs:497-527, :722-815), with
// the argument lists of the Q8_0 pair above:
//   moe_gu_q4k(x, wg, wu, act, idx, K, N)              moe_down_{q5k,q6k}(act, wd, y, idx, wgt, K, N, KSEL)
// f32 activations meet the dequantized weights (the float contract; the CPU path's int8-activation arithmetic is
// what the _dec / _m / _mm / _mt entries above compute).  moe_down_q4k is this library's addition, so that an
// all-Q4_K layer runs under the same contract.
MOE_ROWS_GU_ENTRY(q4k, Q4kW)
MOE_ROWS_DOWN_ENTRY(q4k, Q4kW)
MOE_ROWS_DOWN_ENTRY(q5k, Q5kW)
MOE_ROWS_DOWN_ENTRY(q6k, Q6kW)
