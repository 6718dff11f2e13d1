// Shared device-side vocabulary for the gfx950 kernels: element types, 16-byte
// fragments, MFMA wrappers, wave reductions.  gfx950 (CDNA4) only: 64-wide
// wavefronts, v_mfma_f32_32x32x16_{f16,bf16}, v_mfma_f32_32x32x2_f32.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace aidn {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// Storage element tags.  f16 / bf16 travel as raw 16-bit patterns across the C ABI.
struct f16_t { uint16_t bits; };
struct bf16_t { uint16_t bits; };

constexpr int WAVE = 64;

// Bit reinterpretation through by-value scalars.  (Applying __builtin_bit_cast directly to an element
// of an ext_vector lvalue, e.g. v[i], reads element 0 for every i with this compiler.)
__device__ __forceinline__ float as_f32(uint32_t v) { return __builtin_bit_cast(float, v); }
__device__ __forceinline__ uint32_t as_u32(float v) { return __builtin_bit_cast(uint32_t, v); }

// ------------------------------------------------------------------ conversions
__device__ __forceinline__ float bf16_bits_to_float(uint32_t b) { return as_f32(b << 16); }

// float -> bf16 bits, round-to-nearest-even; NaN keeps sign/payload top bits with the
// quiet bit forced (the rule of the reference's BFloat16.FromFloat,
// src/AiDotNet.Tensors/NumericOperations/BFloat16.cs:64-82).  Integer arithmetic, so the
// result is bit-identical to the host rule for every input.
__device__ __forceinline__ uint32_t float_to_bf16_bits(float f)
{
    uint32_t u = as_u32(f);
    if ((u & 0x7F800000u) == 0x7F800000u && (u & 0x007FFFFFu) != 0u) return (u >> 16) | 0x0040u;
    return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

// float -> IEEE binary16 bits, round-to-nearest-even (v_cvt_f16_f32 under the default
// rounding mode).
__device__ __forceinline__ uint32_t float_to_f16_bits(float f)
{
    _Float16 h = (_Float16)f;
    return (uint32_t)__builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ float f16_bits_to_float(uint32_t b)
{
    return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
}

template <typename T> struct Elem;
template <> struct Elem<float> {
    static constexpr int BYTES = 4;
    static constexpr int PER16 = 4;   // elements per 16-byte fragment
};
template <> struct Elem<f16_t> {
    static constexpr int BYTES = 2;
    static constexpr int PER16 = 8;
    static __device__ __forceinline__ uint32_t narrow(float f) { return float_to_f16_bits(f); }
    static __device__ __forceinline__ float widen(uint32_t b) { return f16_bits_to_float(b); }
};
template <> struct Elem<bf16_t> {
    static constexpr int BYTES = 2;
    static constexpr int PER16 = 8;
    static __device__ __forceinline__ uint32_t narrow(float f) { return float_to_bf16_bits(f); }
    static __device__ __forceinline__ float widen(uint32_t b) { return bf16_bits_to_float(b); }
};

// ------------------------------------------------------------------------- MFMA
// One "fragment step" multiplies a 32 x KS tile of A by a KS x 32 tile of B where each
// lane supplies one 16-byte fragment per operand:
//   lane l, operand A: row  (l % 32), the 16 bytes at k-chunk (l / 32)
//   lane l, operand B: col  (l % 32), the 16 bytes at k-chunk (l / 32)
// 16-bit types: KS = 16, one v_mfma_f32_32x32x16.  fp32: KS = 8, four
// v_mfma_f32_32x32x2_f32 where step s takes element s of each lane's fragment; the
// k index a lane feeds is (4 * (l/32) + s), the same for A and B, so the contraction
// covers all 8 k exactly once.
// Accumulator layout (all 32x32 MFMAs): lane l holds column (l % 32) and rows
// 8*(r/4) + 4*(l/32) + (r%4) for r = 0..15.
template <typename T> struct Mma32;
template <> struct Mma32<f16_t> {
    static constexpr int KS = 16;
    static __device__ __forceinline__ void run(f32x16& acc, const u32x4& a, const u32x4& b)
    {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), acc, 0, 0, 0);
    }
};
template <> struct Mma32<bf16_t> {
    static constexpr int KS = 16;
    static __device__ __forceinline__ void run(f32x16& acc, const u32x4& a, const u32x4& b)
    {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
    }
};
template <> struct Mma32<float> {
    static constexpr int KS = 8;
    static __device__ __forceinline__ void run(f32x16& acc, const u32x4& a, const u32x4& b)
    {
#pragma unroll
        for (int s = 0; s < 4; s++)
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(as_f32(a[s]), as_f32(b[s]), acc, 0, 0, 0);
    }
};

// Row of the 32x32 accumulator that register r of lane-half h holds.
__device__ __forceinline__ int acc_row(int r, int h) { return 8 * (r >> 2) + 4 * h + (r & 3); }

// --------------------------------------------------------- register transposes
// 8x8 transpose of 16-bit elements held as 8 row fragments (row r = in[r], 8 elements
// each) into 8 column fragments (out[c] = column c, elements ordered by row).
__device__ __forceinline__ void transpose8x8_b16(const u32x4 (&in)[8], u32x4 (&out)[8])
{
#pragma unroll
    for (int c = 0; c < 8; c++) {
#pragma unroll
        for (int w = 0; w < 4; w++) {
            uint32_t lo = in[2 * w][c >> 1], hi = in[2 * w + 1][c >> 1];
            // v_perm_b32: selector bytes 0-3 pick from the second operand, 4-7 from the first
            out[c][w] = (c & 1) ? __builtin_amdgcn_perm(hi, lo, 0x07060302u) : __builtin_amdgcn_perm(hi, lo, 0x05040100u);
        }
    }
}
// 4x4 transpose of 32-bit elements (pure register renaming).
__device__ __forceinline__ void transpose4x4_b32(const u32x4 (&in)[4], u32x4 (&out)[4])
{
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
        for (int w = 0; w < 4; w++) out[c][w] = in[w][c];
}

// Pool row of logical key `key` under a block table (vLLM-style paged K/V cache; null table = identity).
__device__ __forceinline__ long long paged_row(const int* __restrict__ bt, int bsz, int key)
{
    if (!bt) return key;
    const int blk = key / bsz;
    return (long long)bt[blk] * bsz + (key - blk * bsz);
}

// ---------------------------------------------------------------- wave helpers
__device__ __forceinline__ float shfl_xor_f(float v, int mask) { return __shfl_xor(v, mask, WAVE); }

// Value held by lane (l ^ 32), through the gfx950 half-wave swap (a VALU operation, no LDS round trip):
// after v_permlane32_swap(a = v, b = v) register a holds the low half's values in both halves and b the
// high half's, so lane l < 32 finds its partner in b and lane l >= 32 in a.
__device__ __forceinline__ void half_swap(float v, float& lo_half, float& hi_half)
{
    uint32_t u = as_u32(v);
    auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    uint32_t a = r[0], b = r[1];
    lo_half = as_f32(a);
    hi_half = as_f32(b);
}
__device__ __forceinline__ float max_with_partner32(float v) { float a, b; half_swap(v, a, b); return fmaxf(a, b); }
__device__ __forceinline__ float sum_with_partner32(float v) { float a, b; half_swap(v, a, b); return a + b; }
// The same between the lanes l and l ^ 16 (v_permlane16_swap: the odd 16-lane rows of one operand change places with the even rows
// of the other, so with both operands v one result holds the even row's value of every row pair and the other the odd row's).
__device__ __forceinline__ void row_swap(float v, float& even_row, float& odd_row)
{
    uint32_t u = as_u32(v);
    auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    uint32_t a = r[0], b = r[1];
    even_row = as_f32(a);
    odd_row = as_f32(b);
}
__device__ __forceinline__ float max_with_partner16(float v) { float a, b; row_swap(v, a, b); return fmaxf(a, b); }
__device__ __forceinline__ float sum_with_partner16(float v) { float a, b; row_swap(v, a, b); return a + b; }

// One interleaved rotary pair: (xe, xo) -> (xe c - xo s, xe s + xo c).  One definition for the stand-alone kernels and for the
// GEMM pass that rotates while it sums, so that both round alike (HipAttentionKernels.cs:958-989 is the reference form).
__device__ __forceinline__ void rope_rotate(float xe, float xo, float c, float s, float& re, float& ro)
{
    // (spelled out as one product and one fused multiply-add each, so that every kernel that calls this rounds the same way
    // whatever the compiler would contract around it)
    re = __builtin_fmaf(xe, c, -(xo * s));
    ro = __builtin_fmaf(xe, s, xo * c);
    // (the fp32 results are made opaque: a caller that narrows them to fp16 would otherwise be compiled to the mixed-precision
    // multiply-add that rounds the exact sum to fp16 once, one caller and not the other, and the two would differ at near-ties)
    asm("" : "+v"(re), "+v"(ro));
}

}  // namespace aidn
