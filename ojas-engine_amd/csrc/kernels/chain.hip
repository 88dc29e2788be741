// Family "chain": the dependent stages of a decode step — q/k/v, o, gate/up, down, the output head, or any other
// sequence of Q4_K matvecs each reading what an earlier one wrote — in ONE launch.
//
//   decode_chain_q4k(ojk_chain_args)        grid = all stages' workgroups, block 256; arguments in ojk_chain.h
//
// Every stage is the arithmetic of the CPU reference's matvec_kq (crates/ojas-cpu/src/cpu_math.rs:1145-1189):
// quant_q8k of the stage's f32 vector (:539-563), then dot_q4k per row (:609-635) — the same lane map, the same
// order of operations and therefore the same bits as quantize_q8k + gemv_q8k_q4k launched one after the other.
// The reference fuses neighbouring projections per launch (crates/ojas-cuda/src/kernels/gemv_q8.rs:229-260); a
// chain of separate launches still pays, per dependent stage, two dispatches (quantizer, matvec), each with the
// chip drained before it and a first round trip to DRAM with nothing in flight.
//
// Here the grid is the concatenation of the stages: for stage s a few quantizer workgroups, then its row
// workgroups (four waves, one or two rows per wave, exactly the separate launch's shape).  The hardware hands
// workgroups out in index order as compute units free up, so the chip stays full across stage borders and the
// load balance is the dispatcher's, as in separate launches.  What one workgroup hands to another travels as a
// pair {value, launch tag}, one 8-byte access past the caches (agent scope: the XCDs' L2s are not coherent with
// each other):
//
//  * a row workgroup stores its results to the caller's vector and, if a later stage reads them, as pairs;
//  * a stage's quantizer workgroups wait until every element of the stage's input carries this launch's tag
//    (an input from outside the launch needs no wait), apply the stage's prologue, quantize 256-element
//    segments into the stage's int8 vector, wait until those stores are acknowledged, and then publish
//    {scale of the segment, tag} — in 64 copies, so that the thousands of waves waiting for them do not all
//    poll one line;
//  * a row wave waits for the {scale, tag} of every segment, then multiplies exactly as the separate launch
//    does.  (Asking for the first weights before the wait — weights never depend on activations — was built
//    and measured: the compute units then fill with waiting workgroups whose requests queue in the memory
//    system, every round trip of the dependency itself takes several times longer behind them, and the chain
//    as a whole loses a few per cent.)
//
// Every wait looks a bounded number of times.  One that gives up sets a host-visible status word and a device-side
// abort word (the other waits stop at their next look at it) and its wave exits; nothing that depends on it
// can complete, so those waits give up too, every wave exits, and the host reports the failure at its next
// synchronisation.  A wait can only be for workgroups with a lower index, and workgroups are handed out in index
// order: whatever a resident workgroup waits for is resident or done.  The bound is there for the case that this
// property of the dispatcher does not hold.
#include "ojk_common.h"
#include "ojk_q4k_dot.h"
#include "ojk_act.h"
#include "ojk_chain.h"

typedef const __attribute__((address_space(4))) ojk_chain_args* ChArgs;
typedef unsigned long long u64;

__device__ __forceinline__ uint ch_sgpr(uint v) { return (uint)__builtin_amdgcn_readfirstlane((int)v); }

// agent-scope accesses: coherent across the XCDs' L2s
__device__ __forceinline__ u64 ch_ld64(const void* p) {
    return __hip_atomic_load((u64*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float ch_ld(const float* p) {
    return __hip_atomic_load((float*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void ch_st(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void ch_st_pair(ojk_chain_pair* p, float v, uint tag) {
    __hip_atomic_store((u64*)p, (u64)__float_as_uint(v) | ((u64)tag << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool ch_aborted(ChArgs a) {
    return ch_sgpr(__hip_atomic_load(a->abort_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) != 0u;
}
__device__ __forceinline__ void ch_give_up(ChArgs a, uint s, uint lane) {
    if (lane == 0) {
        __hip_atomic_store(a->abort_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_store(a->status, s + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}
// One more look allowed?  (`it` counts the looks taken.)
__device__ __forceinline__ bool ch_again(ChArgs a, uint& it, uint cap) {
    if (++it >= cap) return false;
    if ((it & 31u) == 0u && ch_aborted(a)) return false;
    __builtin_amdgcn_s_sleep(8);
    return true;
}

// stacked row -> (tensor, row within it)
__device__ __forceinline__ uint ch_tensor_of(ChArgs a, uint s, uint gr, uint& lr) {
    const uint E0 = a->st[s].ends[0], E1 = a->st[s].ends[1], E2 = a->st[s].ends[2];
    const uint i = gr < E0 ? 0u : gr < E1 ? 1u : gr < E2 ? 2u : 3u;
    lr = gr - (i == 0u ? 0u : i == 1u ? E0 : i == 2u ? E1 : E2);
    return i;
}

// Four consecutive values of segment `seg` for this lane, from a plain vector (two 8-byte loads) or a handed-on
// one (four pairs): the loads go out now, `ch_seg_take` looks at what came back.
struct ChSeg { u64 r[4]; };
__device__ __forceinline__ void ch_seg_issue(const void* src, bool tagged, uint seg, uint lane, ChSeg& o) {
    const size_t e = (size_t)seg * 256u + lane * 4u;
    if (tagged) {
#pragma unroll
        for (int k = 0; k < 4; k++) o.r[k] = ch_ld64((const u64*)src + e + k);
    } else {
        o.r[0] = ch_ld64((const float*)src + e);
        o.r[1] = ch_ld64((const float*)src + e + 2);
    }
}
__device__ __forceinline__ bool ch_seg_take(bool tagged, uint tag, const ChSeg& in, float (&o)[4]) {
    bool ok = true;
    if (tagged) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            o[k] = __uint_as_float((uint)in.r[k]);
            ok = ok && (uint)(in.r[k] >> 32) == tag;
        }
    } else {
        o[0] = __uint_as_float((uint)in.r[0]); o[1] = __uint_as_float((uint)(in.r[0] >> 32));
        o[2] = __uint_as_float((uint)in.r[1]); o[3] = __uint_as_float((uint)(in.r[1] >> 32));
    }
    return ok;
}

// ---------------------------------------------------------------------------------------------------------------
// A quantizer workgroup: OJK_CHAIN_QSEGS segments of the stage's input, one per wave.
__device__ __forceinline__ void ch_quantizer(ChArgs a, uint s, uint q, double* part) {
    const uint tid = threadIdx.x, lane = tid & 63u, wave = ch_sgpr(tid >> 6);
    const uint nsb = a->st[s].K >> 8, pro = a->st[s].prologue, tg = a->st[s].tagged, tag = a->tag, cap = a->spin_cap;
    const bool mul = pro == OJK_CHAIN_X_SILU_MUL || pro == OJK_CHAIN_X_GELU_MUL;
    const bool waits = (tg & 1u) || (mul && (tg & 2u));
    const void* const x = a->st[s].x;
    const void* const x2 = a->st[s].x2;
    unsigned long long* const trace = q == 0u && wave == 0u && lane == 0 ? (unsigned long long*)a->trace : nullptr;
    if (trace) trace[s * OJK_CHAIN_TRACE_EVENTS + OJK_CHAIN_T_QUANT_ENTER] = wall_clock64();
    if (waits && cap == 0u) { ch_give_up(a, s, lane); return; }

    const uint seg0 = q * 4u + wave;
    const bool has0 = seg0 < nsb;
    float v0[4] = {0, 0, 0, 0};
    uint it = 0;
    bool gave_up = false;
    // ---- this wave's own segment (a wave without one still joins the norm's sum below)
    for (;;) {
        ChSeg a0, b0;
        if (has0) ch_seg_issue(x, tg & 1u, seg0, lane, a0);
        if (mul && has0) ch_seg_issue(x2, tg & 2u, seg0, lane, b0);
        bool ok = true;
        if (has0) ok = ch_seg_take(tg & 1u, tag, a0, v0);
        if (mul) {
            const uint act = pro == OJK_CHAIN_X_GELU_MUL ? 1u : 0u;
            float u0[4] = {0, 0, 0, 0};
            if (has0) ok = ch_seg_take(tg & 2u, tag, b0, u0) && ok;
#pragma unroll
            for (int e = 0; e < 4; e++) v0[e] = ffn_act(v0[e], act) * u0[e];
        }
        if (!waits || __all(ok)) break;
        if (!ch_again(a, it, cap)) { gave_up = true; break; }
    }
    if (pro == OJK_CHAIN_X_RMSNORM) {
        // x * (1 / sqrt(mean(x^2) + eps)) * gamma (crates/ojas-cpu/src/cpu_math.rs:456-460).  Every quantizer
        // workgroup of the stage sums the whole vector, in the order rmsnorm_q8k does: a lane the squares of its four
        // values of a segment, the segment's lanes by wave_sum_f64, the segment sums likewise (tree_sum_f64); in f64, rounded once.
        if (tid == 0) part[64] = 0.0;
        __syncthreads();
        for (uint sg = wave; sg < nsb && !gave_up; sg += 8u) {   // two segments of this wave per look
            for (;;) {
                ChSeg t[2];
#pragma unroll
                for (int i = 0; i < 2; i++)
                    if (sg + 4u * (uint)i < nsb) ch_seg_issue(x, tg & 1u, sg + 4u * (uint)i, lane, t[i]);
                bool ok = true;
                float f[2][4];
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    f[i][0] = f[i][1] = f[i][2] = f[i][3] = 0.0f;
                    if (sg + 4u * (uint)i < nsb) ok = ch_seg_take(tg & 1u, tag, t[i], f[i]) && ok;
                }
                if (!(tg & 1u) || __all(ok)) {
#pragma unroll
                    for (int i = 0; i < 2; i++) {
                        double sq = (double)f[i][0] * (double)f[i][0];
                        sq += (double)f[i][1] * (double)f[i][1];
                        sq += (double)f[i][2] * (double)f[i][2];
                        sq += (double)f[i][3] * (double)f[i][3];
                        sq = wave_sum_f64(sq);
                        if (lane == 0 && sg + 4u * (uint)i < nsb) part[sg + 4u * (uint)i] = sq;
                    }
                    break;
                }
                if (!ch_again(a, it, cap)) { gave_up = true; break; }
            }
        }
        if (gave_up && lane == 0) part[64] = -1.0;          // (a sum of squares is never negative)
        __syncthreads();   // all four waves get here, also one whose wait gave up
        if (part[64] < 0.0) gave_up = true;
        const double total = tree_sum_f64(part, nsb, lane);
        const float mean = (float)(total / (double)a->st[s].K);
        const float inv = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(mean, __uint_as_float(a->st[s].eps_bits))));
        const float* gamma = (const float*)x2;
        if (has0) {
            const float4 gm = *(const float4*)(gamma + (size_t)seg0 * 256u + lane * 4u);
            v0[0] = __fmul_rn(__fmul_rn(v0[0], inv), gm.x); v0[1] = __fmul_rn(__fmul_rn(v0[1], inv), gm.y);
            v0[2] = __fmul_rn(__fmul_rn(v0[2], inv), gm.z); v0[3] = __fmul_rn(__fmul_rn(v0[3], inv), gm.w);
        }
    }
    if (gave_up) { ch_give_up(a, s, lane); return; }   // nothing is published: the stage's rows will give up too
    if (trace) trace[s * OJK_CHAIN_TRACE_EVENTS + OJK_CHAIN_T_QUANT_ARRIVED] = wall_clock64();
    // ---- quant_q8k of the two segments: the codes past the caches, then — once they are acknowledged — the scales
    float sc0 = 1.0f;
    auto quantize = [&](const float (&v)[4], uint seg, float& scale) {
        const float amax = wave_max(fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))));
        scale = amax > 0.0f ? __fdiv_rn(amax, 127.0f) : 1.0f;
        const float inv = __fdiv_rn(1.0f, scale);
        const int q0 = (int)sat127(roundf(__fmul_rn(v[0], inv)));
        const int q1 = (int)sat127(roundf(__fmul_rn(v[1], inv)));
        const int q2 = (int)sat127(roundf(__fmul_rn(v[2], inv)));
        const int q3 = (int)sat127(roundf(__fmul_rn(v[3], inv)));
        __hip_atomic_store((uint*)(a->st[s].xq + (size_t)seg * 256u + lane * 4u),
                           (uint)(q0 & 0xFF) | ((uint)(q1 & 0xFF) << 8) | ((uint)(q2 & 0xFF) << 16) | ((uint)(q3 & 0xFF) << 24),
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    if (has0) quantize(v0, seg0, sc0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the codes have been written through
    // lane r writes copy r
    if (has0) ch_st_pair(a->st[s].xs + lane * 64u + seg0, sc0, tag);
    if (trace) trace[s * OJK_CHAIN_TRACE_EVENTS + OJK_CHAIN_T_QUANT_DONE] = wall_clock64();
}

// ---------------------------------------------------------------------------------------------------------------
// A row workgroup: four waves, R rows each — gemv_q8k_q4k's arithmetic.
template <int R>
__device__ __forceinline__ void ch_rows(ChArgs a, uint s, uint rb) {
    const uint tid = threadIdx.x, lane = tid & 63u, wave = ch_sgpr(tid >> 6);
    const uint E3 = a->st[s].ends[3];
    const uint row0 = (rb * 4u + wave) * (uint)R;
    if (row0 >= E3) return;
    const uint nsb = a->st[s].K >> 8, nsteps = (nsb + 7u) >> 3, tag = a->tag, cap = a->spin_cap;
    const uint g = lane >> 3, l = lane & 7u, c = l >> 1;

    const uchar* wr[R];
    float* yr[R];
    ojk_chain_pair* on[R];
    const ojk_chain_pair* ad[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        uint lr;
        const uint i = ch_tensor_of(a, s, min(row0 + (uint)r, E3 - 1u), lr);
        wr[r] = (const uchar*)a->st[s].w[i] + (size_t)lr * nsb * Q4K_BYTES;
        yr[r] = (float*)a->st[s].y[i] + lr;
        on[r] = a->st[s].xchg[i] ? a->st[s].xchg[i] + lr : nullptr;
        ad[r] = a->st[s].addsrc[i] ? a->st[s].addsrc[i] + lr : nullptr;
    }
    if (cap == 0u) { ch_give_up(a, s, lane); return; }
    uint it = 0;
    // ---- an accumulating stage: the old values (written by an earlier stage of this launch: from its pairs)
    float add[R];
#pragma unroll
    for (int r = 0; r < R; r++) add[r] = 0.0f;
    if (a->st[s].accum) {
#pragma unroll
        for (int r = 0; r < R; r++) {
            if (ad[r]) {
                for (;;) {
                    const u64 p = ch_ld64(ad[r]);
                    if (ch_sgpr((uint)(p >> 32)) == tag) { add[r] = __uint_as_float((uint)p); break; }
                    if (!ch_again(a, it, cap)) { ch_give_up(a, s, lane); return; }
                }
            } else {
                add[r] = ch_ld(yr[r]);
            }
        }
    }
    // ---- the input: {scale, tag} of every segment, from the copy this wave looks at; lane i keeps segment i's scale
    float scale;
    {
        const ojk_chain_pair* const mine =
            a->st[s].xs + ((blockIdx.x * 4u + wave) & (OJK_CHAIN_REPLICAS - 1u)) * 64u + min(lane, nsb - 1u);
        for (;;) {
            const u64 p = ch_ld64(mine);
            scale = __uint_as_float((uint)p);
            if (__all((uint)(p >> 32) == tag)) break;
            if (!ch_again(a, it, cap)) { ch_give_up(a, s, lane); return; }
        }
    }
    // ---- the rows
    const signed char* const xq = a->st[s].xq;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.0f;
    for (uint step = 0; step < nsteps; step++) {
        const uint sb = g + 8u * step, sbc = min(sb, nsb - 1u);
        uint4 h[R], q[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uchar* blk = wr[r] + (size_t)sbc * Q4K_BYTES;
            h[r] = *(const uint4*)blk;
            q[r] = *(const uint4*)(blk + 16u + l * 16u);
        }
        Q4kFrag f;
        const signed char* p = xq + (size_t)sbc * 256u + c * 64u + (l & 1u) * 16u;
        f.xl = *(const uint4*)p;
        f.xh = *(const uint4*)(p + 32);
        f.bl = bytesum4(f.xl);
        f.bh = bytesum4(f.xh);
        f.sx = __shfl(scale, (int)sbc);
        if (sb < nsb) {
#pragma unroll
            for (int r = 0; r < R; r++) acc[r] += q4k_lane_dot(h[r], q[r], c, f);
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
        float t = wave_sum(acc[r]);
        if (lane == 0 && row0 + (uint)r < E3) {
            if (a->st[s].accum) t = add[r] + t;
            ch_st(yr[r], t);
            if (on[r]) ch_st_pair(on[r], t, tag);
        }
    }
}

extern "C" __global__ void __launch_bounds__(OJK_CHAIN_THREADS)
decode_chain_q4k(ojk_chain_args in_kernarg) {
    (void)in_kernarg;   // read through the kernarg segment: stages are indexed at run time
    ChArgs a = (ChArgs)__builtin_amdgcn_kernarg_segment_ptr();
    __shared__ double part[65];     // the norm's segment sums; [64]: negative once a wave's wait gave up
    const uint b = blockIdx.x, nst = a->nstages;
    uint s = 0;
    for (uint t = 1; t < nst; t++)
        if (b >= a->st[t].wg_first) s = t;
    const uint local = b - a->st[s].wg_first, nq = a->st[s].n_quant;
    if (local < nq) ch_quantizer(a, s, local, part);
    else if (a->st[s].rows_per_wave == 2u) ch_rows<2>(a, s, local - nq);
    else ch_rows<1>(a, s, local - nq);
}
