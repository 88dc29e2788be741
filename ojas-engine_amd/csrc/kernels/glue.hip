// Family "glue": element-wise helpers around the matmul kernels and two plain streaming kernels
// used to calibrate bandwidth measurements.
//
//   copy_f32_half(x, y, n)   f32 -> f16, round to nearest even  (reference: copy_f32_half,
//                            crates/ojas-cuda/src/kernels/vision.rs:188-189, run before the
//                            split-K GEMM entries)
//   copy_f32_bf16(x, y, n)   f32 -> bf16, round to nearest even
//   copy_bf16_f32(x, y, n)   bf16 -> f32 (exact)
//   copy_bf16_half(x, y, n)  bf16 -> f16, round to nearest even
//   fill_zero_u32(y, n)      y[i] = 0 for n dwords (a fill kernel, safe inside a captured graph)
//   copy_{bf16,f32}_half_zero(x, y, z, n, nz, CB)  the conversion and a zero fill of nz dwords at z in one launch
//   stream_copy_u32x4(x, y, n16)  y = x for n16 16-byte units: a copy of known size
//   stream_read_u32x4(x, y, n16)  reads n16 16-byte units, writes one dword per wave (y: grid*4 dwords)
//   calib_mfma_i8(x, y, iters, mode)   the same for v_mfma_i32_16x16x64_i8 (modes 0 and 1)
//   calib_mfma_f16(x, y, iters, mode)  matrix-pipe calibration: what v_mfma_f32_32x32x16_f16 sustains on the
//                            operands found in x (32 KB: a workgroup's 8 fragments per thread), one wave per SIMD,
//                            16 independent accumulator blocks per wave as in the prefill tile; mode 0 keeps the
//                            fragments in registers, mode 1 reads them back from LDS before every group of 16
//                            MFMAs (4 + 4 reads of 128 bits), mode 2 adds the copies, LDS writes and vector-ALU work
//                            of a dequantizing tile's K step (x then holds 32 KB + 4 MB); y: one dword per thread
#include "ojk_common.h"

// The element-wise kernels are grid-stride loops over groups of 8 elements (128-bit accesses when
// both pointers are 16-byte aligned), plus a scalar tail: any grid of 256-thread blocks is valid.
template <class In, class Out, class F>
__device__ __forceinline__ void map8_at(const In* __restrict__ x, Out* __restrict__ y, uint n, F f, uint t, uint stride) {
    uint done = 0;
    if ((((size_t)x | (size_t)y) & 15u) == 0) {
        const uint n8 = n >> 3;
        for (uint i = t; i < n8; i += stride) {
            In v[8];
            Out o[8];
            if (sizeof(In) == 4) { *(uint4*)v = ((const uint4*)x)[2 * i]; *(uint4*)(v + 4) = ((const uint4*)x)[2 * i + 1]; }
            else *(uint4*)v = ((const uint4*)x)[i];
#pragma unroll
            for (int e = 0; e < 8; e++) o[e] = f(v[e]);
            if (sizeof(Out) == 4) { ((uint4*)y)[2 * i] = *(uint4*)o; ((uint4*)y)[2 * i + 1] = *(uint4*)(o + 4); }
            else ((uint4*)y)[i] = *(uint4*)o;
        }
        done = n8 << 3;
    }
    for (uint i = done + t; i < n; i += stride) y[i] = f(x[i]);
}
template <class In, class Out, class F>
__device__ __forceinline__ void map8(const In* __restrict__ x, Out* __restrict__ y, uint n, F f) {
    map8_at(x, y, n, f, blockIdx.x * 256u + threadIdx.x, gridDim.x * 256u);
}

extern "C" __global__ void __launch_bounds__(256)
copy_f32_half(const float* __restrict__ x, ushort* __restrict__ y, uint n) {
    map8(x, y, n, [](float v) { return __half_as_ushort(__float2half_rn(v)); });
}

extern "C" __global__ void __launch_bounds__(256)
copy_f32_bf16(const float* __restrict__ x, ushort* __restrict__ y, uint n) {
    map8(x, y, n, [](float v) { return f32_to_bf16_bits(v); });
}

extern "C" __global__ void __launch_bounds__(256)
copy_bf16_f32(const ushort* __restrict__ x, float* __restrict__ y, uint n) {
    map8(x, y, n, [](ushort v) { return bf16_bits_to_f32(v); });
}

// bf16 -> f16, round to nearest even (exact for every bf16 value inside f16's normal range)
extern "C" __global__ void __launch_bounds__(256)
copy_bf16_half(const ushort* __restrict__ x, ushort* __restrict__ y, uint n) {
    map8(x, y, n, [](ushort v) { return __half_as_ushort(__float2half_rn(bf16_bits_to_f32(v))); });
}

__device__ __forceinline__ void fill_zero_at(uint* __restrict__ y, uint n, uint t, uint stride) {
    uint done = 0;
    if (((size_t)y & 15u) == 0) {
        const uint n4 = n >> 2;
        for (uint i = t; i < n4; i += stride) ((uint4*)y)[i] = make_uint4(0u, 0u, 0u, 0u);
        done = n4 << 2;
    }
    for (uint i = done + t; i < n; i += stride) y[i] = 0u;
}
extern "C" __global__ void __launch_bounds__(256)
fill_zero_u32(uint* __restrict__ y, uint n) {
    fill_zero_at(y, n, blockIdx.x * 256u + threadIdx.x, gridDim.x * 256u);
}

// The two launches ahead of a split-K tile in one: the first CB workgroups convert n activations to f16, the others
// clear nz dwords of the output the K slices will add into.   copy_{bf16,f32}_half_zero(x, y, z, n, nz, CB), any
// grid with more than CB workgroups.
extern "C" __global__ void __launch_bounds__(256)
copy_bf16_half_zero(const ushort* __restrict__ x, ushort* __restrict__ y, uint* __restrict__ z, uint n, uint nz, uint CB) {
    if (blockIdx.x < CB)
        map8_at(x, y, n, [](ushort v) { return __half_as_ushort(__float2half_rn(bf16_bits_to_f32(v))); },
                blockIdx.x * 256u + threadIdx.x, CB * 256u);
    else fill_zero_at(z, nz, (blockIdx.x - CB) * 256u + threadIdx.x, (gridDim.x - CB) * 256u);
}
extern "C" __global__ void __launch_bounds__(256)
copy_f32_half_zero(const float* __restrict__ x, ushort* __restrict__ y, uint* __restrict__ z, uint n, uint nz, uint CB) {
    if (blockIdx.x < CB)
        map8_at(x, y, n, [](float v) { return __half_as_ushort(__float2half_rn(v)); }, blockIdx.x * 256u + threadIdx.x, CB * 256u);
    else fill_zero_at(z, nz, (blockIdx.x - CB) * 256u + threadIdx.x, (gridDim.x - CB) * 256u);
}

extern "C" __global__ void __launch_bounds__(256)
stream_copy_u32x4(const uint4* __restrict__ x, uint4* __restrict__ y, uint n16) {
    size_t stride = (size_t)gridDim.x * 256u;
    for (size_t i = (size_t)blockIdx.x * 256u + threadIdx.x; i < n16; i += stride) y[i] = x[i];
}

extern "C" __global__ void __launch_bounds__(256)
stream_read_u32x4(const uint4* __restrict__ x, uint* __restrict__ y, uint n16) {
    size_t stride = (size_t)gridDim.x * 256u;
    uint acc = 0;
    for (size_t i = (size_t)blockIdx.x * 256u + threadIdx.x; i < n16; i += stride) {
        uint4 v = x[i];
        acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
    acc = (uint)wave_sum_i32((int)acc);
    if ((threadIdx.x & 63u) == 0) y[blockIdx.x * 4u + (threadIdx.x >> 6)] = acc;
}

typedef _Float16 cal_half8 __attribute__((ext_vector_type(8)));
typedef _Float16 cal_half2 __attribute__((ext_vector_type(2)));
typedef float cal_float16 __attribute__((ext_vector_type(16)));
typedef uint cal_u32x4 __attribute__((ext_vector_type(4)));

// 2 * 32 * 32 * 16 flops per MFMA, 64 per trip, 4 waves per workgroup: flops = grid * 4 * iters * 64 * 32768.
// mode 2 adds, per trip of 64 MFMAs and workgroup, what a 256 x 256 x 64 step of a dequantizing tile moves besides its
// fragment reads: 32 KB copied global -> LDS (walking a 4 MB window behind the operands), 32 KB written to LDS from
// registers, and 160 vector-ALU instructions per thread.
template <int mode>
__device__ __forceinline__ void calib_mfma_body(uint4* tile, const uint4* __restrict__ x, uint* __restrict__ y, uint iters) {
    const uint tid = threadIdx.x, lane = tid & 63u, wave = (uint)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    cal_half8 a[4], b[4];
#pragma unroll
    for (int i = 0; i < 8; i++) tile[i * 256 + tid] = x[i * 256 + tid];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; i++) {
        a[i] = __builtin_bit_cast(cal_half8, tile[i * 256 + tid]);
        b[i] = __builtin_bit_cast(cal_half8, tile[(4 + i) * 256 + tid]);
    }
    cal_float16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) acc[i][j][v] = 0.0f;
    const uint lds0 = (uint)(size_t)(__attribute__((address_space(3))) uchar*)tile;
    const uchar* big = (const uchar*)x + 8u * 256u * 16u;
    cal_half2 va[5];
#pragma unroll
    for (int i = 0; i < 5; i++) va[i] = (cal_half2){(_Float16)(0.001f * (float)(tid + i)), (_Float16)0.5f};
    const cal_half2 vm = {(_Float16)0.999f, (_Float16)1.001f}, vc = {(_Float16)0.0001f, (_Float16)-0.0001f};
    const uint4 w4 = x[tid];
    const cal_u32x4 wv = {w4.x, w4.y, w4.z, w4.w};
    for (uint t = 0; t < iters; t++) {
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            if (mode) {
                // the slot moves with t so that the reads cannot be hoisted out of the loop
                const uint s = (tid + 64u * ((t + ks) & 3u)) & 255u;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    a[i] = __builtin_bit_cast(cal_half8, tile[i * 256 + s]);
                    b[i] = __builtin_bit_cast(cal_half8, tile[(4 + i) * 256 + s]);
                }
            }
            if (mode == 2) {
#pragma unroll
                for (int c = 0; c < 2; c++) {
                    const uint slab = (t * 8u + ks * 2u + c) & 1023u;
                    const uchar* src = big + (size_t)slab * 4096u + wave * 1024u;
                    const uint dst = lds0 + 32768u + (ks * 2 + c) * 4096u + wave * 1024u;
                    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(lane * 16u), "s"(src), "s"(dst) : "memory");
                    const uint wdst = lds0 + 65536u + ((ks * 2 + c) * 256u + tid) * 16u;
                    asm volatile("ds_write_b128 %0, %1" : : "v"(wdst), "v"(wv) : "memory");
                }
            }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[i][j], 0, 0, 0);
                    if (mode == 2) {
                        // 160 per trip: two on every MFMA, a third on every other one
                        va[0] = __builtin_elementwise_fma(va[0], vm, vc);
                        va[1] = __builtin_elementwise_fma(va[1], vm, vc);
                        if (j & 1) va[2 + (i & 1)] = __builtin_elementwise_fma(va[2 + (i & 1)], vm, vc);
                    }
                }
        }
        if (mode == 2) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int v = 0; v < 16; v++) sum += acc[i][j][v];
#pragma unroll
    for (int i = 0; i < 5; i++) sum += (float)va[i][0] + (float)va[i][1];
    y[blockIdx.x * 256u + tid] = __float_as_uint(sum);
}

// The same for the int8 matrix instruction of the prefill tiles in the CPU path's arithmetic: v_mfma_i32_16x16x64_i8,
// 2 * 16 * 16 * 64 operations each, 64 per trip over 16 independent sums; mode 0 operands in registers, mode 1 read
// back from LDS per group of 16.  ops = grid * 4 * iters * 64 * 32768.
typedef int cal_i32x4 __attribute__((ext_vector_type(4)));
template <int mode>
__device__ __forceinline__ void calib_mfma_i8_body(uint4* tile, const uint4* __restrict__ x, uint* __restrict__ y, uint iters) {
    const uint tid = threadIdx.x;
    cal_i32x4 a[4], b[4];
#pragma unroll
    for (int i = 0; i < 8; i++) tile[i * 256 + tid] = x[i * 256 + tid];
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; i++) {
        a[i] = __builtin_bit_cast(cal_i32x4, tile[i * 256 + tid]);
        b[i] = __builtin_bit_cast(cal_i32x4, tile[(4 + i) * 256 + tid]);
    }
    cal_i32x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = (cal_i32x4){0, 0, 0, 0};
    for (uint t = 0; t < iters; t++) {
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            if (mode) {
                const uint s = (tid + 64u * ((t + ks) & 3u)) & 255u;
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    a[i] = __builtin_bit_cast(cal_i32x4, tile[i * 256 + s]);
                    b[i] = __builtin_bit_cast(cal_i32x4, tile[(4 + i) * 256 + s]);
                }
            }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[i], b[j], acc[i][j], 0, 0, 0);
        }
    }
    int sum = 0;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int v = 0; v < 4; v++) sum += acc[i][j][v];
    y[blockIdx.x * 256u + tid] = (uint)sum;
}
extern "C" __global__ void __launch_bounds__(256)
calib_mfma_i8(const uint4* __restrict__ x, uint* __restrict__ y, uint iters, uint mode) {
    __shared__ __attribute__((aligned(1024))) uint4 tile[8 * 256];
    if (mode == 0) calib_mfma_i8_body<0>(tile, x, y, iters);
    else calib_mfma_i8_body<1>(tile, x, y, iters);
}

extern "C" __global__ void __launch_bounds__(256)
calib_mfma_f16(const uint4* __restrict__ x, uint* __restrict__ y, uint iters, uint mode) {
    __shared__ __attribute__((aligned(1024))) uint4 tile[8 * 256 + 2048 + 2048];   // operands | copy target | write target
    if (mode == 0) calib_mfma_body<0>(tile, x, y, iters);
    else if (mode == 1) calib_mfma_body<1>(tile, x, y, iters);
    else calib_mfma_body<2>(tile, x, y, iters);
}
