/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement ("oracle") of the reference's
 * reduced-precision storage conversions.  Nothing in the shipped library
 * links, loads or calls this file; only tests, the smoke check and the
 * bench's cpu_baseline leg do.
 *
 * Pinned by: closed-form bit tests (ties, NaN, Inf, subnormals), an exhaustive
 * sweep of all 65536 half patterns against numpy.float16, and randomized
 * float->half / float->bf16 checks against numpy / torch casts
 * (tests/test_oracle_convert.py).
 */
#include <stdint.h>
#include <string.h>

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* float -> bfloat16, round-to-nearest-even; a NaN keeps its sign and payload's
 * top bits and gets the quiet bit forced on.
 * Follows src/AiDotNet.Tensors/NumericOperations/BFloat16.cs:64-82. */
uint16_t orc_bf16_from_float(float v)
{
    uint32_t bits = f2u(v);
    if ((bits & 0x7F800000u) == 0x7F800000u && (bits & 0x007FFFFFu) != 0)
        return (uint16_t)((bits >> 16) | 0x0040u);
    uint32_t lsb = (bits >> 16) & 1u;
    return (uint16_t)((bits + 0x7FFFu + lsb) >> 16);
}

/* bfloat16 -> float is a 16-bit left shift (lossless).
 * Follows src/AiDotNet.Tensors/NumericOperations/BFloat16.cs:85-90. */
float orc_bf16_to_float(uint16_t h) { return u2f(((uint32_t)h) << 16); }

/* float -> IEEE binary16, round-to-nearest-even.  This is what the reference's
 * `(Half)float` cast does (System.Half is IEEE binary16; used by
 * src/AiDotNet.Tensors/Engines/Simd/HalfKernels.cs:96) and what its device
 * conversion kernel does (`__float2half`,
 * src/AiDotNet.Tensors/Engines/DirectGpu/HIP/Kernels/HipFp16Kernels.cs:27-35). */
uint16_t orc_f16_from_float(float v)
{
    uint32_t x = f2u(v);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t absx = x & 0x7FFFFFFFu;
    if (absx >= 0x7F800000u) {                 /* Inf / NaN */
        if (absx == 0x7F800000u) return (uint16_t)(sign | 0x7C00u);
        /* NaN: keep top mantissa bits, force quiet bit so it stays a NaN */
        return (uint16_t)(sign | 0x7C00u | 0x0200u | ((absx >> 13) & 0x03FFu));
    }
    if (absx >= 0x477FF000u) {                 /* >= 65520 rounds to Inf */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (absx < 0x38800000u) {                  /* below the smallest normal half (2^-14) */
        if (absx < 0x33000000u) return (uint16_t)sign;      /* < 2^-25 -> 0 (2^-25 itself ties to even = 0) */
        /* subnormal half: value = m * 2^-24, m in [0, 1023] */
        int exp = (int)(absx >> 23);                        /* biased float exponent, 102..112 */
        uint32_t man = (absx & 0x007FFFFFu) | 0x00800000u;  /* 24-bit significand */
        int shift = 126 - exp;                              /* 14..24: bits dropped so that result = man >> shift */
        uint32_t q = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);                        /* q == 1024 lands on the smallest normal: correct */
    }
    /* normal range */
    uint32_t exp = ((absx >> 23) - 112u);                   /* rebias 127 -> 15 */
    uint32_t man = absx & 0x007FFFFFu;
    uint32_t q = (exp << 10) | (man >> 13);
    uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++; /* carry into exponent is correct */
    return (uint16_t)(sign | q);
}

/* IEEE binary16 -> float (lossless widen), the `(float)Half` cast of
 * src/AiDotNet.Tensors/Engines/Simd/HalfKernels.cs:79-80. */
float orc_f16_to_float(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x03FFu;
    if (exp == 0x1Fu) return u2f(sign | 0x7F800000u | (man << 13));
    if (exp == 0) {
        if (man == 0) return u2f(sign);
        /* subnormal: normalise */
        int e = -1;
        do { man <<= 1; e++; } while ((man & 0x0400u) == 0);
        man &= 0x03FFu;
        return u2f(sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13));
    }
    return u2f(sign | ((exp + 112u) << 23) | (man << 13));
}

void orc_convert_f32_to_bf16(const float* in, uint16_t* out, long n)
{ for (long i = 0; i < n; i++) out[i] = orc_bf16_from_float(in[i]); }
void orc_convert_bf16_to_f32(const uint16_t* in, float* out, long n)
{ for (long i = 0; i < n; i++) out[i] = orc_bf16_to_float(in[i]); }
void orc_convert_f32_to_f16(const float* in, uint16_t* out, long n)
{ for (long i = 0; i < n; i++) out[i] = orc_f16_from_float(in[i]); }
void orc_convert_f16_to_f32(const uint16_t* in, float* out, long n)
{ for (long i = 0; i < n; i++) out[i] = orc_f16_to_float(in[i]); }

/* Portable input generator restated from the reference's own GPU-vs-CPU test:
 * a PCG-style 32-bit hash mapped to [-0.5, 0.5]
 * (tests/AiDotNet.Tensors.Tests/Engines/DirectGpu/GpuCpuConsistencyTests.cs:100-109).
 * Pure uint32 wrap-around arithmetic, so a future C# run regenerates identical inputs. */
float orc_hash_uniform(uint32_t v)
{
    uint32_t x = v * 747796405u + 2891336453u;
    x = ((x >> ((x >> 28) + 4u)) ^ x) * 277803737u;
    x = (x >> 22) ^ x;
    return (float)(x & 0xFFFFu) / 65535.0f - 0.5f;
}
void orc_fill_hash_uniform(float* out, long n, uint32_t seed)
{ for (long i = 0; i < n; i++) out[i] = orc_hash_uniform((uint32_t)i + seed); }
