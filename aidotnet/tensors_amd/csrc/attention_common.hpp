// Declarations shared by the attention translation units: the kernel argument block, direct-to-LDS loads, packed
// conversions of probabilities.
#pragma once
#include "common.hpp"
#include "launch.hpp"
#include <type_traits>

namespace aidn {

// Division of a 31-bit unsigned number by a divisor fixed at launch: q = (mulhi(x, m) + x) >> s with s = ceil(log2 d),
// m = floor(2^32 (2^s - d) / d) + 1 (two scalar instructions and a shift where the compiler's general sequence takes about 25).
struct FastDiv { uint32_t m, s; };
inline FastDiv make_fastdiv(uint32_t d)
{
    uint32_t s = 0;
    while ((1ull << s) < d) s++;
    return FastDiv{(uint32_t)((((1ull << s) - d) << 32) / d + 1), s};
}
__device__ __forceinline__ uint32_t fastdiv(uint32_t x, FastDiv f) { return (__umulhi(x, f.m) + x) >> f.s; }

struct AttnArgs {
    const void* q; const void* k; const void* v; void* o;
    float* lse; const float* bias; const float* mask;
    int B, H, Hkv, Sq, Sk, D;
    float scale; int causal; int qoff; float softcap; int mask_mode;
    long long bias_bs;
    long long qs[3], ks[3], vs[3], os[3];
    int qtiles;
    int nvb;       // pipelined prefill kernel: virtual blocks (the grid's workgroups take them in turn)
    int alt_from;  // pipelined prefill kernel: first workgroup of the second half of a resident grid (shares its CU with an earlier one)
    FastDiv dgroup, dunits, dqtiles;      // pipelined prefill kernel: H / Hkv, qtiles / 2, qtiles as divisors
    int hgroup;    // general kernel, causal: > 0 heads per group of the workgroup order of a large grid; < 0 the placement of a small one
    // fast kernel, grouped decode: the workgroup's key range is split `split` of nsplit (chunk keys each) and, when part is not
    // null, it stores its unnormalised partial (m, l, O[128]) at part + ((b H_q + head) nsplit + split) * 130 for the merge pass
    int nsplit, chunk; float* part;
    int stream;    // fast kernel: K and V are read once per launch (grouped decode): non-temporal loads
    int stage_out; // fast kernel: fp32 O goes through LDS and is written as whole rows
    int paired;    // fast kernel, causal: a workgroup runs query tile qtiles-1-i and then tile i of a head (equal work for every workgroup)
    int vec_in;    // q/k/v rows are 16-byte aligned and D is a multiple of the 16-byte element count
    int vec_out;
    const int* bt; int bsz; long long bt_bs;   // block table of a paged K/V cache (null = contiguous), block size, batch stride
};

template <typename T> struct Raw2;
template <> struct Raw2<float> { typedef uint32_t type; };
template <> struct Raw2<f16_t> { typedef uint16_t type; };
template <> struct Raw2<bf16_t> { typedef uint16_t type; };

// 16 bytes = PER16 consecutive elements from p; elements at index >= valid read as zero.
template <typename T>
__device__ __forceinline__ u32x4 ld16(const typename Raw2<T>::type* p, int valid, bool vec)
{
    u32x4 v = {0u, 0u, 0u, 0u};
    if (valid <= 0) return v;
    if (vec && valid >= Elem<T>::PER16) return *(const u32x4*)p;
    if (valid >= Elem<T>::PER16) {
        // rows off the 16-byte grid: a whole chunk is still one load, only element-aligned (the hardware takes such loads)
        typedef u32x4 u32x4_a4 __attribute__((aligned(4)));
        typedef u32x4 u32x4_a2 __attribute__((aligned(2)));
        if constexpr (Elem<T>::BYTES == 4) return *(const u32x4_a4*)p;
        else return *(const u32x4_a2*)p;
    }
    if constexpr (Elem<T>::BYTES == 4) {
#pragma unroll
        for (int e = 0; e < 4; e++) if (e < valid) v[e] = p[e];
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) if (e < valid) v[e >> 1] |= ((uint32_t)p[e]) << (16 * (e & 1));
    }
    return v;
}

constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;

// Direct global -> LDS load of 16 bytes per lane: lane i's data lands at LDS address lds_dst + 16 i (lds_dst wave
// uniform).  Issued from inline asm so the compiler does not order later LDS reads behind it; completion is
// awaited explicitly (s_waitcnt vmcnt(0) + barrier) before the tile is read.
__device__ __forceinline__ void attn_dma16(const void* gptr, uint32_t lds_dst)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_dst), "v"(gptr) : "memory");
}
// same, source = wave-uniform base (SGPR pair) + per-lane unsigned 32-bit byte offset
__device__ __forceinline__ void attn_dma16_base(const void* base_uniform, uint32_t lane_off, uint32_t lds_dst)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_dst), "v"(lane_off), "s"(base_uniform) : "memory");
}

// non-temporal forms for a cache that is read once per launch (decode)
__device__ __forceinline__ void attn_dma16_stream(const void* gptr, uint32_t lds_dst)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" ::"s"(lds_dst), "v"(gptr) : "memory");
}
__device__ __forceinline__ void attn_dma16_base_stream(const void* base_uniform, uint32_t lane_off, uint32_t lds_dst)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt" ::"s"(lds_dst), "v"(lane_off), "s"(base_uniform) : "memory");
}

typedef short s16x4a __attribute__((ext_vector_type(4)));

// packed conversions of probabilities and pair sums (shared by both kernels)
template <typename T> __device__ __forceinline__ uint32_t pack2_p(float a, float b);
template <> __device__ __forceinline__ uint32_t pack2_p<f16_t>(float a, float b)
{
    // one packed round-to-nearest-even convert (v_cvt_pk_f16_f32)
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    f2 x = {a, b};
    h2 v = __builtin_convertvector(x, h2);
    return __builtin_bit_cast(uint32_t, v);
}
// acc + lo + hi of a packed pair (one VALU operation)
template <typename T> __device__ __forceinline__ float add_pair(uint32_t packed, float acc);
template <> __device__ __forceinline__ float add_pair<f16_t>(uint32_t packed, float acc)
{
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    const h2 ones = {(_Float16)1.0f, (_Float16)1.0f};
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, packed), ones, acc, false);
}
template <> __device__ __forceinline__ float add_pair<bf16_t>(uint32_t packed, float acc)
{
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    const bf2 ones = {(__bf16)1.0f, (__bf16)1.0f};
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf2, packed), ones, acc, false);
}
template <> __device__ __forceinline__ uint32_t pack2_p<bf16_t>(float a, float b)
{
    // probabilities are finite and non-negative: the hardware round-to-nearest-even convert equals the
    // integer rule of float_to_bf16_bits on them
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    bf2 v = {(__bf16)a, (__bf16)b};
    return __builtin_bit_cast(uint32_t, v);
}


// 16-bit, head dimension 128, plain / causal attention in the software-pipelined form (attention_prefill.hip); kind: 1 fp16, 2 bf16
bool attn_prefill_applies(const AttnArgs& a);
hipError_t launch_attn_prefill(int kind, int out16, AttnArgs a, hipStream_t stream);

}  // namespace aidn
