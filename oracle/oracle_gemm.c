/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement ("oracle") of the reference's GEMM
 * hot path.  Nothing in the shipped library links, loads or calls this file;
 * only tests, the smoke check and the bench's cpu_baseline leg do.
 *
 * What it restates (paths relative to the reference checkout):
 *   - the BLIS-style 5-loop fp32 GEMM with a 6x16 FMA register tile
 *     (src/AiDotNet.Tensors/Engines/Simd/SimdGemm.cs:3198-3323 loop nest,
 *      :3673-3836 panel packing, :3850-3957 macro kernel, :3964-4106 micro kernel,
 *      :3536-3661 2-D tile parallelism, :64-66/:129-130/:151-152 blocking constants);
 *   - the fp16 / bf16 matmuls with fp32 accumulation
 *     (src/AiDotNet.Tensors/Engines/Simd/HalfKernels.cs:35-99,
 *      src/AiDotNet.Tensors/Engines/Simd/BFloat16Kernels.cs:144-211);
 *   - an fp64-accumulated "truth" GEMM used as the error yardstick.
 *
 * Pinned by (tests/test_oracle_gemm.py): dyadic inputs where every summation
 * order is exact (must equal integer arithmetic bit for bit), the reference's
 * literal bf16 known answer [[58,64],[139,154]]
 * (tests/AiDotNet.Tensors.Tests/Engines/Simd/BFloat16KernelsTests.cs:55-68),
 * identity / scaling known answers, the reference's edge shapes (7,13,11),
 * (96,130,80), (37,53,71), (13,17,10), agreement with numpy's float64 matmul,
 * and thread-count independence (bit-identical results for 1 and N threads).
 * Parity unpinned (stated, inside tolerance): the exact bit pattern of large
 * fp32 outputs of the C# build, whose path choice depends on core count and
 * environment flags.
 */
#include <immintrin.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif

float orc_f16_to_float(uint16_t h);
uint16_t orc_f16_from_float(float v);
float orc_bf16_to_float(uint16_t h);
uint16_t orc_bf16_from_float(float v);

enum { MR = 6, NR = 16, KC = 512, NC = 4096, MC_SMALL = 128, MC_LARGE = 192 };

static int imin(int a, int b) { return a < b ? a : b; }
static int imax(int a, int b) { return a > b ? a : b; }

/* Row-block height: 192 when the problem is >= 3e9 FMAs or a medium cube
 * (64e6..1.5e9 FMAs with m == n == k), else 128.  SimdGemm.cs:64-66, 73-83. */
static int choose_mc(int m, int k, int n)
{
    long long work = (long long)m * k * n;
    if (work >= 3000000000LL) return MC_LARGE;
    if (m == n && n == k && work >= 64000000LL && work <= 1500000000LL) return MC_LARGE;
    return MC_SMALL;
}

/* A[ic:ic+mc, pc:pc+kc] -> 6-row panels, element order [panel][p][row]; rows
 * beyond mc are zero filled.  SimdGemm.cs:3673-3752. */
static void pack_a(const float* a, int lda, int transA, float* dst, int ic, int mc, int pc, int kc)
{
    long pos = 0;
    for (int i = 0; i < mc; i += MR) {
        int rows = imin(MR, mc - i);
        for (int p = 0; p < kc; p++) {
            for (int r = 0; r < rows; r++) {
                int row = ic + i + r, col = pc + p;
                dst[pos++] = transA ? a[(long)col * lda + row] : a[(long)row * lda + col];
            }
            for (int r = rows; r < MR; r++) dst[pos++] = 0.0f;
        }
    }
}

/* B[pc:pc+kc, jc:jc+nc] -> 16-column panels, element order [panel][p][col];
 * columns beyond nc are zero filled.  SimdGemm.cs:3772-3836. */
static void pack_b(const float* b, int ldb, int transB, float* dst, int pc, int kc, int jc, int nc)
{
    long pos = 0;
    for (int j = 0; j < nc; j += NR) {
        int cols = imin(NR, nc - j);
        for (int p = 0; p < kc; p++) {
            int row = pc + p;
            if (!transB && cols == NR) {
                memcpy(dst + pos, b + (long)row * ldb + jc + j, NR * sizeof(float));
                pos += NR;
                continue;
            }
            for (int c = 0; c < cols; c++) {
                int col = jc + j + c;
                dst[pos++] = transB ? b[(long)col * ldb + row] : b[(long)row * ldb + col];
            }
            for (int c = cols; c < NR; c++) dst[pos++] = 0.0f;
        }
    }
}

/* 6x16 register tile: 12 eight-lane accumulators start at zero, one fused
 * multiply-add per (row, half) per k in ascending k, then C += acc
 * (load-add-store).  Partial tiles run the same arithmetic on the zero-padded
 * panels and store only the live rows / columns.  SimdGemm.cs:3964-4127
 * (full tile), :3927-3951 (masked edge tile). */
static void micro_6x16(const float* pa, const float* pb, float* c, int ldc, int kc, int rows, int cols)
{
    __m256 acc[MR][2];
    for (int r = 0; r < MR; r++) { acc[r][0] = _mm256_setzero_ps(); acc[r][1] = _mm256_setzero_ps(); }
    for (int p = 0; p < kc; p++) {
        __m256 b0 = _mm256_loadu_ps(pb + (long)p * NR);
        __m256 b1 = _mm256_loadu_ps(pb + (long)p * NR + 8);
        for (int r = 0; r < MR; r++) {
            __m256 av = _mm256_broadcast_ss(pa + (long)p * MR + r);
            acc[r][0] = _mm256_fmadd_ps(av, b0, acc[r][0]);
            acc[r][1] = _mm256_fmadd_ps(av, b1, acc[r][1]);
        }
    }
    if (rows == MR && cols == NR) {
        for (int r = 0; r < MR; r++) {
            float* cr = c + (long)r * ldc;
            _mm256_storeu_ps(cr, _mm256_add_ps(_mm256_loadu_ps(cr), acc[r][0]));
            _mm256_storeu_ps(cr + 8, _mm256_add_ps(_mm256_loadu_ps(cr + 8), acc[r][1]));
        }
    } else {
        float tmp[NR];
        for (int r = 0; r < rows; r++) {
            _mm256_storeu_ps(tmp, acc[r][0]);
            _mm256_storeu_ps(tmp + 8, acc[r][1]);
            float* cr = c + (long)r * ldc;
            for (int j = 0; j < cols; j++) cr[j] = cr[j] + tmp[j];
        }
    }
}

/* All (6-row, 16-col) tiles of one packed A block against one packed B block;
 * column panels outer, row panels inner.  SimdGemm.cs:3850-3957. */
static void macro_kernel(const float* pa, const float* pb, float* c, int mc, int nc, int kc,
                         int ldc, int ic, int jc)
{
    for (int jr = 0; jr < nc; jr += NR) {
        int cols = imin(NR, nc - jr);
        const float* bpanel = pb + (long)(jr / NR) * kc * NR;
        for (int ir = 0; ir < mc; ir += MR) {
            int rows = imin(MR, mc - ir);
            const float* apanel = pa + (long)(ir / MR) * kc * MR;
            micro_6x16(apanel, bpanel, c + (long)(ic + ir) * ldc + jc + jr, ldc, kc, rows, cols);
        }
    }
}

static float* alloc_f32(long n) { void* p = NULL; if (posix_memalign(&p, 64, (size_t)n * 4)) return NULL; return (float*)p; }

/* C += op(A) * op(B) with C row-major [m, n] (ldc = n).  Loop nest
 * jc (4096) -> pc (512) -> ic (Mc): pack, then the macro kernel; with threads > 1
 * the (row block x column sub-block) tiles of one (jc, pc) step are shared out,
 * one thread per C element and a fixed k order, so any thread count gives the
 * same bits.  SimdGemm.cs:3198-3323 and :3536-3661. */
static void sgemm_add(const float* a, int lda, int transA, const float* b, int ldb, int transB,
                      float* c, int m, int k, int n, int threads)
{
    if (m <= 0 || n <= 0 || k <= 0) return;
    int Mc = choose_mc(m, k, n);
    int nrb = (m + Mc - 1) / Mc;
    int mcr = ((Mc + MR - 1) / MR) * MR;
    if (threads < 1) threads = 1;

    for (int jc = 0; jc < n; jc += NC) {
        int nc = imin(NC, n - jc);
        for (int pc = 0; pc < k; pc += KC) {
            int kc = imin(KC, k - pc);
            /* column sub-blocks sized so row blocks x column subs ~ threads, each a
             * multiple of 16 wide, at least 64 wide (SimdGemm.cs:3259-3262, 3549-3557) */
            int want = imax(1, threads / nrb);
            int maxsubs = imax(1, nc / (NR * 4));
            int ncs = imin(want, maxsubs);
            int subw = (nc / ncs / NR) * NR;
            if (subw < NR) { subw = nc; ncs = 1; }
            /* per-sub packed-B region, sized for the widest sub (the last one) */
            int lastw = nc - (ncs - 1) * subw;
            long pb_stride = (long)KC * (((imax(subw, lastw) + NR - 1) / NR) * NR);
            float* pa = alloc_f32((long)nrb * mcr * KC);
            float* pb = alloc_f32(pb_stride * ncs);
            #pragma omp parallel for schedule(dynamic, 1) num_threads(threads) if (threads > 1)
            for (int t = 0; t < nrb + ncs; t++) {
                if (t < nrb) {
                    int ic = t * Mc, mc = imin(Mc, m - ic);
                    pack_a(a, lda, transA, pa + (long)t * mcr * KC, ic, mc, pc, kc);
                } else {
                    int cs = t - nrb, j0 = cs * subw;
                    int w = (cs == ncs - 1) ? nc - j0 : subw;
                    pack_b(b, ldb, transB, pb + pb_stride * cs, pc, kc, jc + j0, w);
                }
            }
            #pragma omp parallel for schedule(dynamic, 1) num_threads(threads) if (threads > 1)
            for (int t = 0; t < nrb * ncs; t++) {
                int r = t / ncs, cs = t % ncs;
                int ic = r * Mc, mc = imin(Mc, m - ic);
                int j0 = cs * subw;
                int w = (cs == ncs - 1) ? nc - j0 : subw;
                macro_kernel(pa + (long)r * mcr * KC, pb + pb_stride * cs, c, mc, w, kc, n, ic, jc + j0);
            }
            free(pa);
            free(pb);
        }
    }
}

/* C = A * B, row-major, overwrite.  The `SimdGemm.Sgemm(a, b, c, m, k, n)` /
 * `SgemmSequential` contract: C is cleared, then accumulated into
 * (SimdGemm.cs:1284-1315, 1345-1353); m, n or k <= 0 leaves C zeroed.
 * Argument order (m, k, n) as in the reference. threads <= 1 is the
 * sequential entry used inside the per-head attention loop. */
void orc_sgemm(const float* a, const float* b, float* c, int m, int k, int n, int threads)
{
    if (m > 0 && n > 0) memset(c, 0, (size_t)m * n * sizeof(float));
    sgemm_add(a, k, 0, b, n, 0, c, m, k, n, threads);
}

/* C = op(A) * op(B) with leading dimensions, the transposed `Sgemm` overload
 * (SimdGemm.cs:1361-1400); C is [m, n] contiguous. */
void orc_sgemm_ex(const float* a, int lda, int transA, const float* b, int ldb, int transB,
                  float* c, int m, int k, int n, int threads)
{
    if (m > 0 && n > 0) memset(c, 0, (size_t)m * n * sizeof(float));
    sgemm_add(a, lda, transA, b, ldb, transB, c, m, k, n, threads);
}

/* The GPU-backend contract `C = alpha * A * B + beta * C`
 * (src/AiDotNet.Tensors/Engines/DirectGpu/IDirectGpuBackend.cs:160-172; transB as in
 * MatMulTransposed :184-203).  The product comes from the restated CPU GEMM; beta == 0
 * must not read C (stale pooled buffers may hold NaN). */
void orc_gemm_alpha_beta(const float* a, const float* b, float* c, int m, int n, int k,
                         float alpha, float beta, int transB, int threads)
{
    float* ab = alloc_f32((long)m * n);
    memset(ab, 0, (size_t)m * n * sizeof(float));
    sgemm_add(a, k, 0, b, transB ? k : n, transB, ab, m, k, n, threads);
    for (long i = 0; i < (long)m * n; i++)
        c[i] = (beta == 0.0f) ? alpha * ab[i] : alpha * ab[i] + beta * c[i];
    free(ab);
}

/* fp64-accumulated truth of float inputs: the yardstick both the restatement and
 * the GPU kernels are measured against (the in-test oracles of
 * tests/AiDotNet.Tensors.Tests/Engines/TensorMatMulSimdFallbackTests.cs:32-96). */
void orc_gemm_f64(const float* a, const float* b, double* c, int m, int k, int n, int transB, int threads)
{
    if (threads < 1) threads = 1;
    #pragma omp parallel for schedule(static) num_threads(threads) if (threads > 1)
    for (int i = 0; i < m; i++) {
        double* acc = c + (long)i * n;
        for (int j = 0; j < n; j++) acc[j] = 0.0;
        if (!transB) {
            for (int p = 0; p < k; p++) {
                double av = a[(long)i * k + p];
                const float* brow = b + (long)p * n;
                for (int j = 0; j < n; j++) acc[j] += av * (double)brow[j];
            }
        } else {
            for (int j = 0; j < n; j++) {
                double s = 0.0;
                for (int p = 0; p < k; p++) s += (double)a[(long)i * k + p] * (double)b[(long)j * k + p];
                acc[j] = s;
            }
        }
    }
}

/* One output element of the reference's 16-bit matmuls: eight fp32 partial sums
 * over k in steps of 8 (FMA), folded lanes (t, t+4), then pairs (0,2)/(1,3), then
 * neighbours; the k % 8 tail is a separate multiply then add.
 * HalfKernels.cs:68-94 and BFloat16Kernels.cs:177-206. */
#pragma GCC push_options
#pragma GCC optimize ("fp-contract=off")
static float dot16(const uint16_t* a, const uint16_t* b, int bstride, int k, float (*widen)(uint16_t))
{
    float acc = 0.0f;
    int kk = 0;
    if (k >= 8) {
        float v[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (; kk + 8 <= k; kk += 8)
            for (int t = 0; t < 8; t++)
                v[t] = fmaf(widen(a[kk + t]), widen(b[(long)(kk + t) * bstride]), v[t]);
        float s0 = v[0] + v[4], s1 = v[1] + v[5], s2 = v[2] + v[6], s3 = v[3] + v[7];
        float t0 = s0 + s2, t1 = s1 + s3;
        acc = t0 + t1;
    }
    for (; kk < k; kk++) {
        float prod = widen(a[kk]) * widen(b[(long)kk * bstride]);
        acc = acc + prod;
    }
    return acc;
}
#pragma GCC pop_options

/* fp16 in, fp32 accumulate.  out16 (RNE-rounded half, `HalfKernels.Matmul`) and/or
 * out32 (the unrounded accumulator: the GemmFp16In32fOut contract,
 * src/AiDotNet.Tensors/Engines/Gpu/IGpuHalfPrecisionBackend.cs:36-48) may be NULL. */
void orc_hgemm(const uint16_t* a, int lda, const uint16_t* b, int ldb,
               uint16_t* out16, float* out32, int ldc, int m, int k, int n, int threads)
{
    if (threads < 1) threads = 1;
    #pragma omp parallel for schedule(static) num_threads(threads) if (threads > 1)
    for (int i = 0; i < m; i++)
        for (int j = 0; j < n; j++) {
            float acc = dot16(a + (long)i * lda, b + j, ldb, k, orc_f16_to_float);
            if (out32) out32[(long)i * ldc + j] = acc;
            if (out16) out16[(long)i * ldc + j] = orc_f16_from_float(acc);
        }
}

/* bf16 in, fp32 accumulate, RNE narrow (`BFloat16Kernels.Matmul`). */
void orc_bf16gemm(const uint16_t* a, int lda, const uint16_t* b, int ldb,
                  uint16_t* out16, float* out32, int ldc, int m, int k, int n, int threads)
{
    if (threads < 1) threads = 1;
    #pragma omp parallel for schedule(static) num_threads(threads) if (threads > 1)
    for (int i = 0; i < m; i++)
        for (int j = 0; j < n; j++) {
            float acc = dot16(a + (long)i * lda, b + j, ldb, k, orc_bf16_to_float);
            if (out32) out32[(long)i * ldc + j] = acc;
            if (out16) out16[(long)i * ldc + j] = orc_bf16_from_float(acc);
        }
}

/* Bias + activation epilogue of FusedLinear: the scalar loop of CpuFusedOperations.ApplyBiasActivationInPlace
 * (src/AiDotNet.Tensors/Helpers/CpuFusedOperations.cs:676-690) with the pointwise functions of its table
 * (:1268-1280; ApplyGelu :1452-1460).  act uses the FusedActivationType numbers (Engines/FusedActivationType.cs:23-70):
 * 0 none, 1 ReLU (NaN-preserving form x < 0 ? 0 : x), 2 GELU tanh form, 3 sigmoid, 4 tanh, 5 leaky ReLU with
 * slope p, 6 swish.  The reference's SIMD variants of None/ReLU/GELU compute the same functions; last-ulp
 * agreement with MathF.Exp / MathF.Tanh is unpinned (libm here). */
static float orc_activation(float x, int act, float p)
{
    switch (act) {
    case 1: return x < 0.0f ? 0.0f : x;
    case 2: { float x3 = x * x * x; float inner = 0.7978845608028654f * (x + 0.044715f * x3); return 0.5f * x * (1.0f + tanhf(inner)); }
    case 3: return 1.0f / (1.0f + expf(-x));
    case 4: return tanhf(x);
    case 5: return x > 0.0f ? x : p * x;
    case 6: return x / (1.0f + expf(-x));
    default: return x;
    }
}

void orc_bias_act_f32(float* c, const float* bias, long m, long n, int act, float p)
{
    for (long i = 0; i < m; i++)
        for (long j = 0; j < n; j++) {
            float v = c[i * n + j];
            if (bias) v += bias[j];
            c[i * n + j] = orc_activation(v, act, p);
        }
}

/* SimdGemm.SgemmNParallelSmallM (src/AiDotNet.Tensors/Engines/Simd/SimdGemm.NParallelSmallM.cs:31-85): C[m,n] (+)= A[m,k] B[k,n]
 * for small m.  Every output column is owned by one worker and is updated once per k in ascending k (one multiply and one
 * add per step, :66-81), so the value of an element does not depend on how the columns are chunked: c = ((c0 + a0 b0) + a1 b1) + ...
 * cleared != 0 starts from 0 (overwrite), otherwise from the existing C (accumulate). */
void orc_sgemm_small_m(const float* a, int lda, const float* b, int ldb, float* c, int m, int k, int n, int cleared)
{
    if (m <= 0 || k <= 0 || n <= 0) return;
#pragma omp parallel for schedule(static)
    for (int j0 = 0; j0 < n; j0 += 64) {
        int j1 = imin(n, j0 + 64);
        for (int i = 0; i < m; i++) {
            float* crow = c + (long)i * n;
            if (cleared) for (int j = j0; j < j1; j++) crow[j] = 0.0f;
            for (int p = 0; p < k; p++) {
                float av = a[(long)i * lda + p];
                const float* brow = b + (long)p * ldb;
                for (int j = j0; j < j1; j++) crow[j] = crow[j] + av * brow[j];
            }
        }
    }
}

int orc_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
