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

// Interleaved rotary position embedding (GPT-NeoX / LLaMA / GGML form): the pair (2i, 2i+1) of row r is rotated by the
// angle of absolute position startPosition + r % seqLen; cos / sin caches are fp32 [maxSeq, headDim / 2].
// Replaces rope_interleaved (src/AiDotNet.Tensors/Engines/DirectGpu/HIP/Kernels/HipAttentionKernels.cs:958-989, one thread
// per pair).  HBM-bound; one thread per pair with 8-byte (fp32) or 4-byte (16-bit) accesses, output may alias input.
template <typename T>
__global__ __launch_bounds__(256) void rope_interleaved_kernel(const void* __restrict__ in, const float* __restrict__ cosc,
                                                               const float* __restrict__ sinc, void* out,
                                                               long long rows, int headDim, int seqLen, int startPosition)
{
    const int half = headDim >> 1;
    const long long total = rows * half;
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long g = (long long)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += stride) {
        const long long row = g / half;
        const int i = (int)(g - row * half);
        const long long pos = startPosition + row % seqLen;
        const float c = cosc[pos * half + i], sn = sinc[pos * half + i];
        float xe, xo;
        if constexpr (Elem<T>::BYTES == 4) {
            u32x2 v = ((const u32x2*)in)[g];
            xe = as_f32(v[0]); xo = as_f32(v[1]);
        } else {
            uint32_t v = ((const uint32_t*)in)[g];
            xe = Elem<T>::widen(v & 0xFFFFu); xo = Elem<T>::widen(v >> 16);
        }
        float re, ro;
        rope_rotate(xe, xo, c, sn, re, ro);
        if constexpr (Elem<T>::BYTES == 4) ((u32x2*)out)[g] = u32x2{as_u32(re), as_u32(ro)};
        else ((uint32_t*)out)[g] = Elem<T>::narrow(re) | (Elem<T>::narrow(ro) << 16);
    }
}

// The same with 16 bytes per thread (two fp32 pairs or four 16-bit pairs) and vector loads of the cos / sin rows: for head
// dimensions that are a multiple of 4 (fp32) / 8 (16-bit) and 16-byte aligned buffers.  One thread per pair moves 8 or 4 bytes
// per access and reaches 4.7 (fp32) / 3.4 (bf16) TB/s of read + write traffic on a 2 GiB tensor.
template <typename T>
__global__ __launch_bounds__(256) void rope_interleaved_vec_kernel(const void* in, const float* __restrict__ cosc,
                                                                   const float* __restrict__ sinc, void* out,
                                                                   long long rows, int headDim, int seqLen, int startPosition)
{
    constexpr int NP = Elem<T>::BYTES == 4 ? 2 : 4;          // pairs per 16 bytes
    const int half = headDim >> 1;
    const int per_row = half / NP;
    const long long total = rows * per_row;
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long g = (long long)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += stride) {
        const long long row = g / per_row;
        const int i = (int)(g - row * per_row) * NP;
        const long long pos = startPosition + row % seqLen;
        const u32x4 v = ((const u32x4*)in)[g];
        u32x4 o;
        if constexpr (Elem<T>::BYTES == 4) {
            const u32x2 c = *(const u32x2*)(cosc + pos * half + i), sn = *(const u32x2*)(sinc + pos * half + i);
#pragma unroll
            for (int p = 0; p < 2; p++) {
                const float xe = as_f32(v[2 * p]), xo = as_f32(v[2 * p + 1]), cc = as_f32(c[p]), ss = as_f32(sn[p]);
                float re, ro;
                rope_rotate(xe, xo, cc, ss, re, ro);
                o[2 * p] = as_u32(re);
                o[2 * p + 1] = as_u32(ro);
            }
        } else {
            const u32x4 c = *(const u32x4*)(cosc + pos * half + i), sn = *(const u32x4*)(sinc + pos * half + i);
#pragma unroll
            for (int p = 0; p < 4; p++) {
                const float xe = Elem<T>::widen(v[p] & 0xFFFFu), xo = Elem<T>::widen(v[p] >> 16), cc = as_f32(c[p]), ss = as_f32(sn[p]);
                float re, ro;
                rope_rotate(xe, xo, cc, ss, re, ro);
                o[p] = Elem<T>::narrow(re) | (Elem<T>::narrow(ro) << 16);
            }
        }
        ((u32x4*)out)[g] = o;
    }
}

// The same rotation over the first `cols` columns of every row of a dense 16-bit [M, N] matrix, in place (the columns are heads of
// headDim elements side by side: what a projection GEMM writes); row m takes the angle of position startPosition + m % seqLen.
template <typename T>
__global__ __launch_bounds__(256) void rope_cols_kernel(uint16_t* __restrict__ C, const float* __restrict__ cosc, const float* __restrict__ sinc,
                                                        int M, int N, int cols, int headDim, int seqLen, int startPosition)
{
    const int half = headDim >> 1, pairs = cols >> 1;
    const long long total = (long long)M * pairs;
    for (long long g = (long long)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += (long long)gridDim.x * blockDim.x) {
        const int m = (int)(g / pairs), col = 2 * (int)(g - (long long)m * pairs);
        const int i = (col % headDim) >> 1;
        const long long pos = startPosition + m % seqLen;
        uint32_t* p = (uint32_t*)(C + (long long)m * N + col);
        const uint32_t v = *p;
        float re, ro;
        rope_rotate(Elem<T>::widen(v & 0xFFFFu), Elem<T>::widen(v >> 16), cosc[pos * half + i], sinc[pos * half + i], re, ro);
        *p = Elem<T>::narrow(re) | (Elem<T>::narrow(ro) << 16);
    }
}

hipError_t rope_cols16(hipStream_t stream, int kind, uint16_t* C, const float* cosc, const float* sinc, int M, int N, int cols, int headDim,
                       int seqLen, int startPosition)
{
    const long long total = (long long)M * (cols / 2);
    if (total <= 0) return hipSuccess;
    const unsigned grid = (unsigned)((total + 255) / 256 > 256 * 32 ? 256 * 32 : (total + 255) / 256);
    if (kind == 1) hipLaunchKernelGGL(rope_cols_kernel<f16_t>, dim3(grid), dim3(256), 0, stream, C, cosc, sinc, M, N, cols, headDim, seqLen, startPosition);
    else if (kind == 2) hipLaunchKernelGGL(rope_cols_kernel<bf16_t>, dim3(grid), dim3(256), 0, stream, C, cosc, sinc, M, N, cols, headDim, seqLen, startPosition);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

// kind: 0 fp32, 1 fp16, 2 bf16
hipError_t rope_interleaved(hipStream_t stream, int kind, const void* in, const float* cosc, const float* sinc, void* out,
                            long long rows, int headDim, int seqLen, int startPosition)
{
    long long pairs = rows * (headDim / 2);
    if (pairs <= 0) return hipSuccess;
    const int np = kind == 0 ? 2 : 4;
    const bool aligned = ((((uintptr_t)in) | ((uintptr_t)out) | ((uintptr_t)cosc) | ((uintptr_t)sinc)) & 15u) == 0;
    if (aligned && (headDim / 2) % np == 0 && (kind == 0 || kind == 1 || kind == 2)) {
        const long long work = pairs / np;
        unsigned grid = (unsigned)((work + 255) / 256 > 256 * 32 ? 256 * 32 : (work + 255) / 256);
        if (kind == 0) hipLaunchKernelGGL(rope_interleaved_vec_kernel<float>, dim3(grid), dim3(256), 0, stream, in, cosc, sinc, out, rows, headDim, seqLen, startPosition);
        else if (kind == 1) hipLaunchKernelGGL(rope_interleaved_vec_kernel<f16_t>, dim3(grid), dim3(256), 0, stream, in, cosc, sinc, out, rows, headDim, seqLen, startPosition);
        else hipLaunchKernelGGL(rope_interleaved_vec_kernel<bf16_t>, dim3(grid), dim3(256), 0, stream, in, cosc, sinc, out, rows, headDim, seqLen, startPosition);
        return hipGetLastError();
    }
    unsigned grid = (unsigned)((pairs + 255) / 256 > 256 * 32 ? 256 * 32 : (pairs + 255) / 256);
    if (kind == 0) hipLaunchKernelGGL(rope_interleaved_kernel<float>, dim3(grid), dim3(256), 0, stream, in, cosc, sinc, out, rows, headDim, seqLen, startPosition);
    else if (kind == 1) hipLaunchKernelGGL(rope_interleaved_kernel<f16_t>, dim3(grid), dim3(256), 0, stream, in, cosc, sinc, out, rows, headDim, seqLen, startPosition);
    else if (kind == 2) hipLaunchKernelGGL(rope_interleaved_kernel<bf16_t>, dim3(grid), dim3(256), 0, stream, in, cosc, sinc, out, rows, headDim, seqLen, startPosition);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

}  // namespace aidn
