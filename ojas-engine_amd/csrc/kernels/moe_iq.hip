// Family "moe_iq": expert products over IQ4_XS and IQ4_NL rows, f32 activations.
//
// The reference's IQ expert kernels by their own names and argument lists
// (crates/ojas-cuda/src/kernels/moe_iq.rs:64-112; the expert table crates/ojas-core/src/quant_src.rs:168-193):
//   moe_gu_<fmt>(x, wg, wu, act, idx, K, N)             grid [ceil(N/8), KSEL, tokens], block 256
//       act[j][n] = silu(gate_e . x) * (up_e . x),  e = idx[j]
//   moe_down_<fmt>(act, wd, y, idx, wgt, K, N, KSEL)    grid [1 .. ceil(N/4), tokens, 1], block 256
//       y[n] += sum_j wgt[j] * (down_e . act[j])        (accumulates onto y)
// for <fmt> = iq4xs and iq4nl — the streamed models keep IQ4_XS gate/up and IQ4_NL down tensors; the table
// also lists moe_down_iq4xs, and both roles of both formats cost nothing more here.  The raw rows meet f32
// activations as dot_iq4xs / dot_iq4nl do (crates/ojas-cpu/src/cpu_math.rs:943-967, :993-1010).
//
// Two things a one-token caller of the reference's launch does not see: the last grid dimension walks
// tokens (token t reads x + t K, idx + t KSEL, wgt + t KSEL and writes act + t KSEL N, y + t N), and a
// trailing constant E, appended by the dispatcher from the extent of the expert tensors, bounds the routed
// indices: a slot whose index is E or more contributes zeros instead of reading past the tensors.
// Rows of the down launch are grid-stride (4 per workgroup and step), so the reference's ceil(N/8)
// workgroups are a valid grid.
//
// The grid-codebook experts of the same table ride the same bodies over the traits of ojk_iq_grid_rows.h:
//   moe_gu_iq3s, moe_gu_iq3s_slots(x, arena_g, arena_u, act, off_g, off_u, K, N)    (moe_iq.rs:173-191; IQ3_S gate/up with
//   IQ4_NL down is the combination the streamed models ship in), moe_gu_iq2xxs, moe_down_iq2xxs, moe_down_iq3xxs,
//   moe_gu_iq2s (the table's remaining IQ rows).
#include "ojk_moe_rows.h"
#include "ojk_iq_grid_rows.h"

#define MOE_IQ_ENTRIES(FMT, W) MOE_ROWS_GU_ENTRY(FMT, W) MOE_ROWS_DOWN_ENTRY(FMT, W)
MOE_IQ_ENTRIES(iq4xs, Iq4xsW)
MOE_IQ_ENTRIES(iq4nl, Iq4nlW)
// (their workgroups expand the codebook into LDS before the rows)
#define MOE_GRID_GU_ENTRY(FMT, W)                                                                           \
    extern "C" __global__ void __launch_bounds__(256) moe_gu_##FMT(                                         \
        const float* x, const uchar* wg, const uchar* wu, float* act, const uint* idx, uint K, uint N,      \
        uint E) { W::init(); __syncthreads(); moe_gu_rows<W>(x, wg, wu, act, idx, K, N, E); }
#define MOE_GRID_GU_SLOTS_ENTRY(FMT, W)                                                                     \
    extern "C" __global__ void __launch_bounds__(256) moe_gu_##FMT##_slots(                                 \
        const float* x, const uchar* arena_g, const uchar* arena_u, float* act, const uint* off_g,          \
        const uint* off_u, uint K, uint N, uint LIM_G, uint LIM_U) {                                        \
        W::init(); __syncthreads();                                                                         \
        moe_gu_rows_slots<W>(x, arena_g, arena_u, act, off_g, off_u, K, N, LIM_G, LIM_U); }
#define MOE_GRID_DOWN_ENTRY(FMT, W)                                                                         \
    extern "C" __global__ void __launch_bounds__(256) moe_down_##FMT(                                       \
        const float* act, const uchar* wd, float* y, const uint* idx, const float* wgt, uint K, uint N,     \
        uint KSEL, uint E) { W::init(); __syncthreads(); moe_down_rows<W>(act, wd, y, idx, wgt, K, N, KSEL, E); }
MOE_GRID_GU_ENTRY(iq3s, Iq3sW)
MOE_GRID_GU_SLOTS_ENTRY(iq3s, Iq3sW)
MOE_GRID_GU_ENTRY(iq2xxs, Iq2xxsW)
MOE_GRID_DOWN_ENTRY(iq2xxs, Iq2xxsW)
MOE_GRID_DOWN_ENTRY(iq3xxs, Iq3xxsW)
MOE_GRID_GU_ENTRY(iq2s, Iq2sW)
