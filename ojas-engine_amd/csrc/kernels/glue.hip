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
//   stream_copy_u32x4(x, y, n16)  y = x for n16 16-byte units: a copy of known size
//   stream_read_u32x4(x, y, n16)  reads n16 16-byte units, writes one dword per wave (y: grid*4 dwords)
#include "ojk_common.h"

// The element-wise kernels are grid-stride loops over groups of 8 elements (128-bit accesses when
// both pointers are 16-byte aligned), plus a scalar tail: any grid of 256-thread blocks is valid.
template <class In, class Out, class F>
__device__ __forceinline__ void map8(const In* __restrict__ x, Out* __restrict__ y, uint n, F f) {
    const uint stride = gridDim.x * 256u, t = blockIdx.x * 256u + threadIdx.x;
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

extern "C" __global__ void __launch_bounds__(256)
fill_zero_u32(uint* __restrict__ y, uint n) {
    const uint stride = gridDim.x * 256u, t = blockIdx.x * 256u + threadIdx.x;
    uint done = 0;
    if (((size_t)y & 15u) == 0) {
        const uint n4 = n >> 2;
        for (uint i = t; i < n4; i += stride) ((uint4*)y)[i] = make_uint4(0u, 0u, 0u, 0u);
        done = n4 << 2;
    }
    for (uint i = done + t; i < n; i += stride) y[i] = 0u;
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
