// Q6_K pieces for the int8 matrix cores, shared by the few-token kernels (family "gemv_q8k") and the 128-token
// tile (family "gemm_q8k").
#pragma once
#include "ojk_common.h"

__device__ __forceinline__ long q6k_signed8(uint ql0, uint ql1, uint qh0, uint qh1, int Q) {
    const uint M4 = 0x0F0F0F0Fu, H2 = 0x30303030u;
    const uint lo0 = Q < 2 ? ql0 & M4 : (ql0 >> 4) & M4, lo1 = Q < 2 ? ql1 & M4 : (ql1 >> 4) & M4;
    const uint hi0 = Q == 0 ? (qh0 << 4) & H2 : Q == 1 ? (qh0 << 2) & H2 : Q == 2 ? qh0 & H2 : (qh0 >> 2) & H2;
    const uint hi1 = Q == 0 ? (qh1 << 4) & H2 : Q == 1 ? (qh1 << 2) & H2 : Q == 2 ? qh1 & H2 : (qh1 >> 2) & H2;
    // code in 0..63 -> code - 32 as int8, bytewise: + 96 cannot carry, the flip of bit 7 subtracts 128
    const uint c0 = ((lo0 | hi0) + 0x60606060u) ^ 0x80808080u, c1 = ((lo1 | hi1) + 0x60606060u) ^ 0x80808080u;
    return (long)(((unsigned long)c1 << 32) | c0);
}

// A super-block is 210 bytes, so a lane's 8-byte pieces sit at even or odd multiples of two
// bytes.  With sixteen rows per load instruction, 8-byte loads that are not dword aligned cost
// the memory pipeline more than their size (measured: 217 -> 161 us for this kernel); these read
// the three aligned dwords around a piece and shift (sh = 0 or 16 bits, v_alignbit).  The
// streaming kernels' 16-byte pieces measured the other way round and stay unaligned loads.
__device__ __forceinline__ u32x2_a2 q6k_ld8(const uchar* a4, uint sh) {   // a4: piece address rounded down to 4
    const uint* p = (const uint*)a4;
    const uint d0 = p[0], d1 = p[1], d2 = p[2];
    u32x2_a2 r;
    r.x = __builtin_amdgcn_alignbit(d1, d0, sh);
    r.y = __builtin_amdgcn_alignbit(d2, d1, sh);
    return r;
}
