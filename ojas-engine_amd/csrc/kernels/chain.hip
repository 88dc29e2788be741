// Family "chain": the dependent stages of a decode step — q/k/v, o, gate/up, down, the output head, or any other
// sequence of Q4_K matvecs each reading what an earlier one wrote — in ONE launch.
//
//   decode_chain_q4k(ojk_chain_args)        grid = compute units, block 1024; arguments in ojk_chain.h
//
// Every stage is the arithmetic of the CPU reference's matvec_kq (crates/ojas-cpu/src/cpu_math.rs:1145-1189):
// quant_q8k of the stage's f32 vector (:539-563), then dot_q4k per row (:609-635) — the same lane map, the same
// order of operations and therefore the same bits as quantize_q8k + gemv_q8k_q4k launched one after the other.
// The reference fuses neighbouring projections per launch (crates/ojas-cuda/src/kernels/gemv_q8.rs:229-260); a
// chain of separate launches still pays, per dependent stage, a dispatch, a quantizer launch and the first round
// trip to DRAM with nothing in flight.  Here the grid is one resident workgroup per compute unit and stays for
// the whole chain:
//
//  * Weights never depend on activations.  Each wave walks one list of units (two 8-super-block steps of
//    weights per lane) across all stages and keeps CH_D units of 16-byte loads in flight in registers, across
//    stage borders too.  Vector memory operations return in order, so when a wave turns to the next stage's
//    input, that input arrives behind the weights the wave has already asked for: memory stays busy while the
//    dependency is resolved, and the stage starts with its first units in registers.
//  * A result that a later stage reads travels as a pair {value, launch tag}, stored and loaded as one 8-byte
//    access past the caches (agent scope, `sc1`: the XCDs' L2s are not coherent with each other).  A stage's
//    input is complete when every element carries this launch's tag; a wave polls its share of the vector
//    (one to four 256-element segments) until it does, a bounded number of times.  No counters, no waiting for
//    stores to be acknowledged, no barrier among workgroups other than the data itself: the arithmetic of stage
//    s + 1 starts only after every row of stage s that it reads has arrived.
//  * The input is quantized by every workgroup into its own LDS.
//  * A wait that gives up sets a host-visible status word and a device-side abort word (the other waits stop
//    at their next look at it), the workgroup skips the remaining arithmetic, every wave exits, and the host
//    reports the failure at its next synchronisation.
//
// The launch tag comes from eight device-side counters: workgroup b adds one to counter b % 8 when it starts and
// divides what it gets by the number of workgroups that share the counter.  Launches of one device run one after
// the other, so all workgroups of a launch compute the same tag and no two launches share one.
#include "ojk_common.h"
#include "ojk_q4k_dot.h"
#include "ojk_act.h"
#include "ojk_chain.h"

#define CH_D 2                     // units in flight per wave
#define CH_SEG 288u                // LDS bytes per 256 quantized activations (fragment reads fall in distinct banks)
#define CH_NSEG (OJK_CHAIN_MAX_K / 256u)
#define CH_XSEG 4                  // segments of the input vector a wave quantizes at most

typedef const __attribute__((address_space(4))) ojk_chain_args* ChArgs;
typedef unsigned long long u64;

// A unit: two 8-super-block steps of weights per lane.  In a stage with at least two rows per wave they are the
// same step of two neighbouring rows (the activation fragment is read once for both); in a smaller stage they are
// two consecutive steps of one row, so that every wave of the chip has a row.
struct ChUnit { uint4 h[2], q[2]; };
struct ChView {
    uint nsb, nsteps, E3;
    uint rpw;      // rows per unit: 2, or 1 in a small stage
    uint upg;      // units per row group
    uint ngrp;     // row groups of this wave
    uint nU, nUpad;
};

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

// What wave `gw` of `NW` owns in stage s: row groups gw, gw + NW, ... (a group = rpw neighbouring rows), each
// `upg` units; the count is padded to a multiple of CH_D (at least CH_D) so that a unit's place in the register
// ring does not depend on the stage.
__device__ __forceinline__ ChView ch_view(ChArgs a, uint s, uint gw, uint NW) {
    ChView v;
    if (s < a->nstages) {
        v.E3 = a->st[s].ends[3];
        v.nsb = a->st[s].K >> 8;
        v.nsteps = (v.nsb + 7u) >> 3;
        v.rpw = (v.E3 + 1u) / 2u < NW ? 1u : 2u;
        v.upg = v.rpw == 2u ? v.nsteps : (v.nsteps + 1u) >> 1;
        const uint G = (v.E3 + v.rpw - 1u) / v.rpw;
        v.ngrp = gw < G ? (G - 1u - gw) / NW + 1u : 0u;
        v.nU = v.ngrp * v.upg;
        v.nUpad = max((v.nU + CH_D - 1u) / CH_D * CH_D, (uint)CH_D);
    } else {
        v.E3 = 1u; v.nsb = 1u; v.nsteps = 1u; v.rpw = 2u; v.upg = 1u; v.ngrp = 0u; v.nU = 0u; v.nUpad = CH_D;
    }
    return v;
}

// stacked row -> (tensor, row within it)
__device__ __forceinline__ uint ch_tensor_of(ChArgs a, uint s, uint gr, uint& lr) {
    const uint E0 = a->st[s].ends[0], E1 = a->st[s].ends[1], E2 = a->st[s].ends[2];
    const uint i = gr < E0 ? 0u : gr < E1 ? 1u : gr < E2 ? 2u : 3u;
    lr = gr - (i == 0u ? 0u : i == 1u ? E0 : i == 2u ? E1 : E2);
    return i;
}

extern "C" __global__ void __launch_bounds__(OJK_CHAIN_THREADS)
decode_chain_q4k(ojk_chain_args in_kernarg) {
    (void)in_kernarg;   // read through the kernarg segment: stages are indexed at run time
    ChArgs a = (ChArgs)__builtin_amdgcn_kernarg_segment_ptr();
    // More than half of the 160 KB: the dispatcher cannot put two of these workgroups on one compute unit and
    // leave another empty.
    __shared__ __attribute__((aligned(16))) uchar lds[84u * 1024u];
    signed char* const sx_all = (signed char*)lds;                          // 2 x CH_NSEG * CH_SEG
    float* const ss_all = (float*)(lds + 2u * CH_NSEG * CH_SEG);            // 2 x CH_NSEG
    double* const part = (double*)(ss_all + 2u * CH_NSEG);                  // OJK_CHAIN_WAVES
    uint* const s_dead = (uint*)(part + OJK_CHAIN_WAVES);   // two words
    uint* const s_tag = s_dead + 2;

    const uint tid = threadIdx.x, lane = tid & 63u;
    const uint wave = ch_sgpr(tid >> 6);
    const uint b = blockIdx.x, nwg = gridDim.x;
    const uint NW = nwg * OJK_CHAIN_WAVES, gw = b * OJK_CHAIN_WAVES + wave;
    const uint g = lane >> 3, l = lane & 7u, c = l >> 1;
    const uint nst = a->nstages;
    uint* const sync = a->sync;
    if (tid == 0) s_dead[0] = s_dead[1] = 0u;   // one word per stage parity: a wave ahead by a stage writes the other one
    unsigned long long* const trace = (unsigned long long*)a->trace;
    auto stamp = [&](uint s, uint ev) {   // the workgroup's first wave
        if (trace && wave == 0u && lane == 0)
            trace[((size_t)b * OJK_CHAIN_MAX_STAGES + s) * OJK_CHAIN_TRACE_EVENTS + ev] = wall_clock64();
    };

    // ---- this launch's tag (asked for first, needed when the first results are handed on)
    u64 ticket = 0;
    if (nst > 1u && tid == 0)
        ticket = __hip_atomic_fetch_add((u64*)(sync + OJK_CHAIN_SYNC_TICKET(b & 7u)), (u64)1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);

    // ---- the look-ahead cursor: which unit the next 16-byte loads belong to
    uint fs = 0, fu = 0, fst = 0, fjj = 0;
    ChView FV = ch_view(a, 0, gw, NW);
    const uchar* frw[2];
    frw[0] = frw[1] = (const uchar*)a->st[0].w[0];
    ChUnit ring[CH_D];

    // The loads are issued on every call, whatever the cursor says, so that the number of loads in flight — what
    // the waits before a unit's first use count — never depends on a branch.  A call without a unit behind it
    // (padding, the end of the chain) reads one 16-byte piece of the last row it saw, the same in every lane.
    auto fetch = [&](ChUnit& slot, bool hold) {
        const bool valid = !hold && fs < nst && fu < FV.nU;
        if (valid && fst == 0u) {
            const uint row0 = (fjj * NW + gw) * FV.rpw;
#pragma unroll
            for (uint r = 0; r < 2u; r++) {
                uint lr;
                const uint i = ch_tensor_of(a, fs, min(row0 + (FV.rpw == 2u ? r : 0u), FV.E3 - 1u), lr);
                frw[r] = (const uchar*)a->st[fs].w[i] + (size_t)lr * FV.nsb * Q4K_BYTES;
            }
        }
        // step of each half: the same for two rows, consecutive for one
        const uint st0 = FV.rpw == 2u ? fst : 2u * fst, st1 = FV.rpw == 2u ? fst : 2u * fst + 1u;
        const uint h0 = valid ? __umul24(min(g + 8u * st0, FV.nsb - 1u), Q4K_BYTES) : 0u;
        const uint h1 = valid ? __umul24(min(g + 8u * st1, FV.nsb - 1u), Q4K_BYTES) : 0u;
        const uint qo = valid ? 16u + l * 16u : 0u;
        slot.h[0] = *(const uint4*)(frw[0] + h0);
        slot.q[0] = *(const uint4*)(frw[0] + (h0 + qo));
        slot.h[1] = *(const uint4*)(frw[1] + h1);
        slot.q[1] = *(const uint4*)(frw[1] + (h1 + qo));
        if (valid && ++fst == FV.upg) { fst = 0u; fjj++; }
        if (!hold && ++fu == FV.nUpad) {
            fs++; fu = 0u; fst = 0u; fjj = 0u;
            FV = ch_view(a, fs, gw, NW);
        }
    };

    // ---- a stage's input.  Wave w owns segments w, w + 16, ...; a lane holds four consecutive values of each.
    // They are fetched two segments (and their second operands) at a time: plain vectors as two 8-byte loads
    // per lane and segment, handed-on vectors as four {value, tag} pairs.  (Segments past the vector are not
    // read: every workgroup reads the same few lines past the caches, and redundant requests for them queue
    // at one memory channel.)
    float xv[CH_XSEG][4], xw[2][4];
    u64 raw[2][4];   // two segments of one vector, or one segment of two (a product prologue)
    uint tag = 0u;
    auto is_mul = [&](uint s) {
        const uint pro = a->st[s].prologue;
        return pro == OJK_CHAIN_X_SILU_MUL || pro == OJK_CHAIN_X_GELU_MUL;
    };
    auto raw_issue = [&](const void* src, bool tagged, uint seg, u64 (&r)[4]) {
        const size_t e = (size_t)seg * 256u + lane * 4u;
        if (tagged) {
#pragma unroll
            for (int k = 0; k < 4; k++) r[k] = ch_ld64((const u64*)src + e + k);
        } else {
            r[0] = ch_ld64((const float*)src + e);
            r[1] = ch_ld64((const float*)src + e + 2);
        }
    };
    // raw -> values; false if a handed-on value has not arrived yet
    auto raw_take = [&](bool tagged, const u64 (&r)[4], float (&o)[4]) -> bool {
        bool ok = true;
        if (tagged) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                o[k] = __uint_as_float((uint)r[k]);
                ok = ok && (uint)(r[k] >> 32) == tag;
            }
        } else {
            o[0] = __uint_as_float((uint)r[0]); o[1] = __uint_as_float((uint)(r[0] >> 32));
            o[2] = __uint_as_float((uint)r[1]); o[3] = __uint_as_float((uint)(r[1] >> 32));
        }
        return ok;
    };
    // Segments `first` (and `first + 1`, unless the prologue is a product) of this wave's share.
    auto batch_issue = [&](uint s, uint nsb, uint first) {
        const uint tg = a->st[s].tagged;
        const uint seg0 = wave + OJK_CHAIN_WAVES * first, seg1 = seg0 + OJK_CHAIN_WAVES;
        if (is_mul(s)) {
            if (seg0 < nsb) {
                raw_issue(a->st[s].x, tg & 1u, seg0, raw[0]);
                raw_issue(a->st[s].x2, tg & 2u, seg0, raw[1]);
            }
        } else {
            if (seg0 < nsb) raw_issue(a->st[s].x, tg & 1u, seg0, raw[0]);
            if (seg1 < nsb) raw_issue(a->st[s].x, tg & 1u, seg1, raw[1]);
        }
    };
    auto batch_take = [&](uint s, uint nsb, uint first, float (&dst0)[4], float (&dst1)[4]) -> bool {
        const uint tg = a->st[s].tagged;
        const uint seg0 = wave + OJK_CHAIN_WAVES * first, seg1 = seg0 + OJK_CHAIN_WAVES;
        bool ok = true;
        if (is_mul(s)) {
            if (seg0 < nsb) {
                ok = raw_take(tg & 1u, raw[0], dst0);
                ok = raw_take(tg & 2u, raw[1], xw[0]) && ok;
                const uint act = a->st[s].prologue == OJK_CHAIN_X_GELU_MUL ? 1u : 0u;
#pragma unroll
                for (int e = 0; e < 4; e++) dst0[e] = ffn_act(dst0[e], act) * xw[0][e];
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) dst0[e] = 0.0f;
            }
        } else {
            if (seg0 < nsb) ok = raw_take(tg & 1u, raw[0], dst0);
            else {
#pragma unroll
                for (int e = 0; e < 4; e++) dst0[e] = 0.0f;
            }
            if (seg1 < nsb) ok = raw_take(tg & 1u, raw[1], dst1) && ok;
            else {
#pragma unroll
                for (int e = 0; e < 4; e++) dst1[e] = 0.0f;
            }
        }
        return __all(ok);
    };
    // One batch: fetch it; while a handed-on part is missing, watch ONE of its elements (every workgroup waits for
    // the same few lines, and whole-segment polls from all of them starve the very stores they wait for at that
    // memory channel), then fetch again — a bounded number of looks in all; false if the wait gave up.
    auto batch_wait = [&](uint s, uint nsb, uint first, bool issued, float (&dst0)[4], float (&dst1)[4]) -> bool {
        const uint cap = a->spin_cap;
        const bool waits = (a->st[s].tagged & 1u) || ((a->st[s].tagged & 2u) && is_mul(s));
        if (!issued) batch_issue(s, nsb, first);
        bool ok = batch_take(s, nsb, first, dst0, dst1);
        if (!waits) return true;
        if (cap == 0u) return false;
        // the element watched: the last one of the batch's last segment, of the vector that is handed on
        const uint seg0 = wave + OJK_CHAIN_WAVES * first, seg1 = seg0 + OJK_CHAIN_WAVES;
        const uint segw = (!is_mul(s) && seg1 < nsb) ? seg1 : min(seg0, nsb - 1u);
        const u64* const watch = (const u64*)((a->st[s].tagged & 1u) ? a->st[s].x : a->st[s].x2) + (size_t)segw * 256u + 255u;
        uint it = 1u;
        while (!ok) {
            for (;; it++) {
                if (it >= cap) return false;
                if ((it & 63u) == 0u &&
                    ch_sgpr(__hip_atomic_load(sync + OJK_CHAIN_SYNC_ABORT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)))
                    return false;
                __builtin_amdgcn_s_sleep(4);
                if ((uint)(ch_ld64(watch) >> 32) == tag) break;   // the same address in every lane: one request
            }
            batch_issue(s, nsb, first);
            ok = batch_take(s, nsb, first, dst0, dst1);
            it++;
        }
        return true;
    };
    // RMS norm over the workgroup, then f32 -> int8 per 256 into the stage's LDS buffer
    auto input_quantize = [&](uint s, uint nsb, signed char* sx, float* ss) {
        if (a->st[s].prologue == OJK_CHAIN_X_RMSNORM) {
            // mean of squares in f64, rounded once (as rmsnorm_q8k does; the reference sums in f32,
            // crates/ojas-cpu/src/cpu_math.rs:456-460)
            const float* gamma = (const float*)a->st[s].x2;
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const uint seg = min(wave + OJK_CHAIN_WAVES * (uint)i, nsb - 1u);
                const float4 t = *(const float4*)(gamma + (size_t)seg * 256u + lane * 4u);
                xw[i][0] = t.x; xw[i][1] = t.y; xw[i][2] = t.z; xw[i][3] = t.w;
            }
            double sq = 0.0;
#pragma unroll
            for (int i = 0; i < CH_XSEG; i++)
#pragma unroll
                for (int e = 0; e < 4; e++) sq += (double)xv[i][e] * (double)xv[i][e];   // (segments past the vector hold zeros)
            for (int off = 32; off > 0; off >>= 1) {
                const long bits = __double_as_longlong(sq);
                const int lo = __shfl_xor((int)bits, off), hi = __shfl_xor((int)(bits >> 32), off);
                sq += __longlong_as_double(((long)hi << 32) | (unsigned int)lo);
            }
            if (lane == 0) part[wave] = sq;
            __syncthreads();
            double tot = 0.0;
#pragma unroll
            for (int w4 = 0; w4 < 4; w4++) tot += (part[w4] + part[w4 + 4]) + (part[w4 + 8] + part[w4 + 12]);
            const float mean = (float)(tot / (double)a->st[s].K);
            const float inv = __fdiv_rn(1.0f, __fsqrt_rn(__fadd_rn(mean, __uint_as_float(a->st[s].eps_bits))));
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int e = 0; e < 4; e++) xv[i][e] = __fmul_rn(__fmul_rn(xv[i][e], inv), xw[i][e]);
            if (nsb > 2u * OJK_CHAIN_WAVES) {
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    const uint seg = min(wave + OJK_CHAIN_WAVES * (2u + (uint)i), nsb - 1u);
                    const float4 t = *(const float4*)(gamma + (size_t)seg * 256u + lane * 4u);
                    xv[2 + i][0] = __fmul_rn(__fmul_rn(xv[2 + i][0], inv), t.x);
                    xv[2 + i][1] = __fmul_rn(__fmul_rn(xv[2 + i][1], inv), t.y);
                    xv[2 + i][2] = __fmul_rn(__fmul_rn(xv[2 + i][2], inv), t.z);
                    xv[2 + i][3] = __fmul_rn(__fmul_rn(xv[2 + i][3], inv), t.w);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < CH_XSEG; i++) {
            const uint seg = wave + OJK_CHAIN_WAVES * (uint)i;
            if (seg < nsb) {
                const float amax = wave_max(fmaxf(fmaxf(fabsf(xv[i][0]), fabsf(xv[i][1])), fmaxf(fabsf(xv[i][2]), fabsf(xv[i][3]))));
                const float scale = amax > 0.0f ? __fdiv_rn(amax, 127.0f) : 1.0f;
                const float inv = __fdiv_rn(1.0f, scale);
                const int q0 = (int)sat127(roundf(__fmul_rn(xv[i][0], inv)));
                const int q1 = (int)sat127(roundf(__fmul_rn(xv[i][1], inv)));
                const int q2 = (int)sat127(roundf(__fmul_rn(xv[i][2], inv)));
                const int q3 = (int)sat127(roundf(__fmul_rn(xv[i][3], inv)));
                *(uint*)(sx + seg * CH_SEG + lane * 4u) =
                    (uint)(q0 & 0xFF) | ((uint)(q1 & 0xFF) << 8) | ((uint)(q2 & 0xFF) << 16) | ((uint)(q3 & 0xFF) << 24);
                if (lane == 0) ss[seg] = scale;
            }
        }
    };

    // The first stage's input is requested before the first weights: loads return in order, and the vector would
    // otherwise wait behind a ring-full of them.
    batch_issue(0, FV.nsb, 0u);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < CH_D; j++) fetch(ring[j], false);

    // the workgroups sharing this one's counter drew tickets t * members .. t * members + members - 1 in launch t
    if (tid == 0) *s_tag = (uint)(ticket / ((nwg - (b & 7u) + 7u) / 8u)) + 1u;

    for (uint s = 0; s < nst; s++) {
        const ChView UV = ch_view(a, s, gw, NW);
        signed char* const sx = sx_all + (s & 1u) * (CH_NSEG * CH_SEG);
        float* const ss = ss_all + (s & 1u) * CH_NSEG;
        stamp(s, OJK_CHAIN_T_ENTER);
        // ---- the input: wait (bounded) until this wave's segments have arrived
        bool arrived;
        if (is_mul(s)) {   // a segment (of both vectors) at a time
            arrived = batch_wait(s, UV.nsb, 0u, s == 0u, xv[0], xv[0]);
            if (arrived) arrived = batch_wait(s, UV.nsb, 1u, false, xv[1], xv[1]);
            if (arrived) arrived = batch_wait(s, UV.nsb, 2u, false, xv[2], xv[2]);
            if (arrived) arrived = batch_wait(s, UV.nsb, 3u, false, xv[3], xv[3]);
        } else {
            arrived = batch_wait(s, UV.nsb, 0u, s == 0u, xv[0], xv[1]);
            if (arrived) arrived = batch_wait(s, UV.nsb, 2u, false, xv[2], xv[3]);
        }
        if (!arrived && lane == 0) {
            s_dead[s & 1u] = s + 1u;
            __hip_atomic_store(sync + OJK_CHAIN_SYNC_ABORT, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(a->status, s + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
        stamp(s, OJK_CHAIN_T_ARRIVED);
        input_quantize(s, UV.nsb, sx, ss);
        __syncthreads();
        if (s == 0u) tag = *s_tag;
        if (s_dead[s & 1u]) break;
        stamp(s, OJK_CHAIN_T_INPUT);

        // ---- the rows
        const bool acc_stage = a->st[s].accum != 0u;
        uint ust = 0u, ujj = 0u;
        float acc0 = 0.0f, acc1 = 0.0f, add0 = 0.0f, add1 = 0.0f;
        auto frag_at = [&](uint sb) {
            Q4kFrag f;
            const signed char* p = sx + sb * CH_SEG + c * 64u + (l & 1u) * 16u;
            f.xl = *(const uint4*)p;
            f.xh = *(const uint4*)(p + 32);
            f.bl = bytesum4(f.xl);
            f.bh = bytesum4(f.xh);
            f.sx = ss[sb];
            return f;
        };
        // one finished row: to the caller's vector and, if a later stage reads it, onward with the launch's tag
        auto publish = [&](uint row, float t, float addend) {
            if (lane == 0 && row < UV.E3) {
                uint lr;
                const uint i = ch_tensor_of(a, s, row, lr);
                if (acc_stage) t = addend + t;
                ch_st((float*)a->st[s].y[i] + lr, t);
                ojk_chain_pair* const on = a->st[s].xchg[i];
                if (on) ch_st_pair(on + lr, t, tag);
            }
        };
        for (uint u = 0; u < UV.nUpad; u += CH_D) {
#pragma unroll
            for (int j = 0; j < CH_D; j++) {
                if (u + (uint)j < UV.nU) {
                    const uint row0 = (ujj * NW + gw) * UV.rpw;
                    if (acc_stage && ust == 0u && lane == 0) {   // the old values, asked for a whole group ahead of their use
                        uint lr;
                        uint i = ch_tensor_of(a, s, min(row0, UV.E3 - 1u), lr);
                        add0 = ch_ld((const float*)a->st[s].y[i] + lr);
                        if (UV.rpw == 2u) {
                            i = ch_tensor_of(a, s, min(row0 + 1u, UV.E3 - 1u), lr);
                            add1 = ch_ld((const float*)a->st[s].y[i] + lr);
                        }
                    }
                    if (UV.rpw == 2u) {
                        const uint sb = g + 8u * ust;
                        if (sb < UV.nsb) {
                            const Q4kFrag f = frag_at(sb);
                            acc0 += q4k_lane_dot(ring[j].h[0], ring[j].q[0], c, f);
                            acc1 += q4k_lane_dot(ring[j].h[1], ring[j].q[1], c, f);
                        }
                    } else {
                        const uint sb = g + 16u * ust;
                        if (sb < UV.nsb) acc0 += q4k_lane_dot(ring[j].h[0], ring[j].q[0], c, frag_at(sb));
                        if (sb + 8u < UV.nsb) acc0 += q4k_lane_dot(ring[j].h[1], ring[j].q[1], c, frag_at(sb + 8u));
                    }
                    if (++ust == UV.upg) {
                        ust = 0u;
                        publish(row0, wave_sum(acc0), add0);
                        if (UV.rpw == 2u) publish(row0 + 1u, wave_sum(acc1), add1);
                        acc0 = acc1 = 0.0f;
                        ujj++;
                    }
                }
                // What belongs to the next stage is held back until every wave of the workgroup has stored its last
                // rows: the compute unit's memory pipeline is one queue, and a store behind the other waves'
                // look-ahead is a result the whole chip waits for.
                fetch(ring[j], fs != s);
            }
        }
        stamp(s, OJK_CHAIN_T_ROWS);
        if (s + 1u < nst) {
            __syncthreads();
#pragma unroll
            for (int j = 0; j < CH_D; j++) fetch(ring[j], false);
        }
    }
}
