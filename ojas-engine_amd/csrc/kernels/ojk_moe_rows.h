// Expert products over raw rows with f32 activations, shared by the families "moe" and "moe_iq": templates over the
// row traits of ojk_rows.h and ojk_iq_grid_rows.h.
//   moe_gu_rows:    act[j][n] = silu(gate_e . x) * (up_e . x),  e = idx[j]      grid [ceil(N/8), KSEL, tokens] x 256
//   moe_down_rows:  y[n] += sum_j wgt[j] * (down_e . act[j])                     grid [1 .. ceil(N/4), tokens, 1] x 256
// A slot whose expert index is E or more contributes zeros instead of reading past the tensors.
#pragma once
#include "ojk_common.h"
#include "ojk_rows.h"

// The rows of one (token, slot): ge / ue point at the slot's gate and up expert (N rows each), nu = the row's units,
// or 0 for a slot that contributes zeros.
template <class W>
__device__ __forceinline__ void moe_gu_rows_at(const float* __restrict__ xt, const uchar* __restrict__ ge,
                                               const uchar* __restrict__ ue, float* __restrict__ out, uint K, uint N,
                                               uint nu) {
    const uint lane = threadIdx.x & 63u;
    const uint row0 = (blockIdx.x * 4u + (threadIdx.x >> 6)) * 2u;
    if (row0 >= N) return;
    const size_t rb = (size_t)W::units(K) * W::BYTES;
    const uchar* g0 = ge + (size_t)row0 * rb;
    const uchar* u0 = ue + (size_t)row0 * rb;
    const size_t r1 = row0 + 1u < N ? rb : 0;        // the last odd row is computed twice, stored once
    float ag[2] = {0.0f, 0.0f}, au[2] = {0.0f, 0.0f};
    for (uint u = W::unit_of(lane); u < nu; u += W::STEP) {
        const typename W::Frag fg0 = W::load(g0, u, lane), fg1 = W::load(g0 + r1, u, lane);
        const typename W::Frag fu0 = W::load(u0, u, lane), fu1 = W::load(u0 + r1, u, lane);
        const float* xp = xt + (size_t)u * W::x_unit(0) + W::x_off(lane);
        const float4 x0 = *(const float4*)xp, x1 = *(const float4*)(xp + W::XGAP);
        const float xsum = sum4(x0) + sum4(x1);
        ag[0] += W::dot(fg0, lane, x0, x1, xsum);
        ag[1] += W::dot(fg1, lane, x0, x1, xsum);
        au[0] += W::dot(fu0, lane, x0, x1, xsum);
        au[1] += W::dot(fu1, lane, x0, x1, xsum);
    }
#pragma unroll
    for (int r = 0; r < 2; r++) {
        const float gs = wave_sum(ag[r]), us = wave_sum(au[r]);
        if (lane == 0 && row0 + r < N) out[row0 + r] = (gs / (1.0f + expf(-gs))) * us;
    }
}

template <class W>
__device__ __forceinline__ void moe_gu_rows(const float* __restrict__ x, const uchar* __restrict__ wg,
                                            const uchar* __restrict__ wu, float* __restrict__ act,
                                            const uint* __restrict__ idx, uint K, uint N, uint E) {
    const uint j = blockIdx.y, t = blockIdx.z, ksel = gridDim.y;
    const uint e = idx[t * ksel + j];
    const size_t eb = (size_t)N * W::units(K) * W::BYTES;
    moe_gu_rows_at<W>(x + (size_t)t * K, wg + (size_t)e * eb, wu + (size_t)e * eb, act + ((size_t)t * ksel + j) * N, K, N,
                      e < E ? W::units(K) : 0u);
}

// Streamed experts: one u32 byte offset per (token, slot) into a cache arena instead of an expert index
// (crates/ojas-cuda/src/kernels/moe_iq.rs:181-191); offsets are rounded down to the blocks' two-byte alignment and
// clamped to LIM, the last offset at which a whole expert still fits its arena.
template <class W>
__device__ __forceinline__ void moe_gu_rows_slots(const float* __restrict__ x, const uchar* __restrict__ arena_g,
                                                  const uchar* __restrict__ arena_u, float* __restrict__ act,
                                                  const uint* __restrict__ off_g, const uint* __restrict__ off_u, uint K,
                                                  uint N, uint LIM_G, uint LIM_U) {
    const uint j = blockIdx.y, t = blockIdx.z, ksel = gridDim.y;
    const uint og = min(off_g[t * ksel + j] & ~1u, LIM_G), ou = min(off_u[t * ksel + j] & ~1u, LIM_U);
    moe_gu_rows_at<W>(x + (size_t)t * K, arena_g + og, arena_u + ou, act + ((size_t)t * ksel + j) * N, K, N, W::units(K));
}

// A workgroup owns four rows at a time (rows grid-stride over the workgroups); its four waves take the slots
// j = wave, wave + 4, ... and meet in LDS, where the partial sums are added in wave order onto y: an expert
// row is short, so the slots are the parallelism that fills the chip at one token.
template <class W>
__device__ __forceinline__ void moe_down_rows(const float* __restrict__ act, const uchar* __restrict__ wd,
                                              float* __restrict__ y, const uint* __restrict__ idx,
                                              const float* __restrict__ wgt, uint K, uint N, uint KSEL, uint E) {
    __shared__ float part[4][4];
    const uint lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint t = blockIdx.y;
    const uint nu = W::units(K);
    const size_t rb = (size_t)nu * W::BYTES;
    for (uint row0 = blockIdx.x * 4u; row0 < N; row0 += gridDim.x * 4u) {
        float res[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (uint j = wave; j < KSEL; j += 4u) {
            const uint e = idx[t * KSEL + j];
            if (e >= E) continue;
            const float wj = wgt[t * KSEL + j];
            const float* xr = act + ((size_t)t * KSEL + j) * K;
            float a[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            for (uint u = W::unit_of(lane); u < nu; u += W::STEP) {
                typename W::Frag f[4];
#pragma unroll
                for (int r = 0; r < 4; r++) f[r] = W::load(wd + ((size_t)e * N + min(row0 + (uint)r, N - 1u)) * rb, u, lane);
                const float* xp = xr + (size_t)u * W::x_unit(0) + W::x_off(lane);
                const float4 x0 = *(const float4*)xp, x1 = *(const float4*)(xp + W::XGAP);
                const float xsum = sum4(x0) + sum4(x1);
#pragma unroll
                for (int r = 0; r < 4; r++) a[r] += W::dot(f[r], lane, x0, x1, xsum);
            }
#pragma unroll
            for (int r = 0; r < 4; r++) res[r] += wj * wave_sum(a[r]);
        }
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < 4; r++) part[wave][r] = res[r];
        }
        __syncthreads();
        if (threadIdx.x < 4u && row0 + threadIdx.x < N)
            y[(size_t)t * N + row0 + threadIdx.x] += ((part[0][threadIdx.x] + part[1][threadIdx.x]) + part[2][threadIdx.x]) + part[3][threadIdx.x];
        __syncthreads();
    }
}

#define MOE_ROWS_GU_ENTRY(FMT, W)                                                                           \
    extern "C" __global__ void __launch_bounds__(256) moe_gu_##FMT(                                         \
        const float* x, const uchar* wg, const uchar* wu, float* act, const uint* idx, uint K, uint N,      \
        uint E) { moe_gu_rows<W>(x, wg, wu, act, idx, K, N, E); }
#define MOE_ROWS_GU_SLOTS_ENTRY(FMT, W)                                                                     \
    extern "C" __global__ void __launch_bounds__(256) moe_gu_##FMT##_slots(                                 \
        const float* x, const uchar* arena_g, const uchar* arena_u, float* act, const uint* off_g,          \
        const uint* off_u, uint K, uint N, uint LIM_G, uint LIM_U) {                                        \
        moe_gu_rows_slots<W>(x, arena_g, arena_u, act, off_g, off_u, K, N, LIM_G, LIM_U); }
#define MOE_ROWS_DOWN_ENTRY(FMT, W)                                                                         \
    extern "C" __global__ void __launch_bounds__(256) moe_down_##FMT(                                       \
        const float* act, const uchar* wd, float* y, const uint* idx, const float* wgt, uint K, uint N,     \
        uint KSEL, uint E) { moe_down_rows<W>(act, wd, y, idx, wgt, K, N, KSEL, E); }
