// Storage conversions fp32 <-> fp16 / bf16 (round-to-nearest-even narrows).
// Replaces ConvertToFp16 / ConvertToFp32 of the reference backend
// (src/AiDotNet.Tensors/Engines/DirectGpu/HIP/HipBackend.cs:11942-11981, kernels
// Kernels/HipFp16Kernels.cs:27-48: one element per thread); bf16 follows
// src/AiDotNet.Tensors/NumericOperations/BFloat16.cs:64-90.  HBM-bound: each thread moves
// 8 elements (32 B in / 16 B out or the reverse) with 128-bit accesses, grid-stride.
#include "common.hpp"
#include "launch.hpp"

namespace aidn {

template <typename T>
__global__ __launch_bounds__(256) void narrow_kernel(const float* __restrict__ in, uint16_t* __restrict__ out, long long n, int vec_ok)
{
    long long nvec = vec_ok ? n / 8 : 0;
    long long stride = (long long)gridDim.x * blockDim.x;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += stride) {
        u32x4 a = ((const u32x4*)in)[2 * i], b = ((const u32x4*)in)[2 * i + 1];
        u32x4 o;
#pragma unroll
        for (int w = 0; w < 2; w++) {
            o[w] = Elem<T>::narrow(as_f32(a[2 * w])) | (Elem<T>::narrow(as_f32(a[2 * w + 1])) << 16);
            o[w + 2] = Elem<T>::narrow(as_f32(b[2 * w])) | (Elem<T>::narrow(as_f32(b[2 * w + 1])) << 16);
        }
        ((u32x4*)out)[i] = o;
    }
    for (long long i = nvec * 8 + (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        out[i] = (uint16_t)Elem<T>::narrow(in[i]);
}

template <typename T>
__global__ __launch_bounds__(256) void widen_kernel(const uint16_t* __restrict__ in, float* __restrict__ out, long long n, int vec_ok)
{
    long long nvec = vec_ok ? n / 8 : 0;
    long long stride = (long long)gridDim.x * blockDim.x;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += stride) {
        u32x4 v = ((const u32x4*)in)[i];
        u32x4 a, b;
#pragma unroll
        for (int w = 0; w < 2; w++) {
            a[2 * w] = as_u32(Elem<T>::widen(v[w] & 0xFFFFu));
            a[2 * w + 1] = as_u32(Elem<T>::widen(v[w] >> 16));
            b[2 * w] = as_u32(Elem<T>::widen(v[w + 2] & 0xFFFFu));
            b[2 * w + 1] = as_u32(Elem<T>::widen(v[w + 2] >> 16));
        }
        ((u32x4*)out)[2 * i] = a;
        ((u32x4*)out)[2 * i + 1] = b;
    }
    for (long long i = nvec * 8 + (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        out[i] = Elem<T>::widen(in[i]);
}

hipError_t convert(hipStream_t stream, int kind, const void* in, void* out, long long n)
{
    if (n <= 0) return hipSuccess;
    int vec_ok = ((((uintptr_t)in) | ((uintptr_t)out)) & 15u) == 0;
    long long work = (n + 7) / 8;
    unsigned grid = (unsigned)((work + 255) / 256);
    if (grid > 256u * 16u) grid = 256u * 16u;
    if (grid == 0) grid = 1;
    switch (kind) {
    case 0: hipLaunchKernelGGL(narrow_kernel<f16_t>, dim3(grid), dim3(256), 0, stream, (const float*)in, (uint16_t*)out, n, vec_ok); break;
    case 1: hipLaunchKernelGGL(widen_kernel<f16_t>, dim3(grid), dim3(256), 0, stream, (const uint16_t*)in, (float*)out, n, vec_ok); break;
    case 2: hipLaunchKernelGGL(narrow_kernel<bf16_t>, dim3(grid), dim3(256), 0, stream, (const float*)in, (uint16_t*)out, n, vec_ok); break;
    case 3: hipLaunchKernelGGL(widen_kernel<bf16_t>, dim3(grid), dim3(256), 0, stream, (const uint16_t*)in, (float*)out, n, vec_ok); break;
    default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace aidn
