/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatements of the reference's secondary GEMM / attention paths: the code
 * the C# build actually runs for some shapes instead of the tiled SimdGemm / FlashAttentionFloat path that
 * oracle_gemm.c and oracle_attention.c restate.  Nothing in the shipped library links, loads or calls this file.
 *
 * What it restates (paths relative to the reference checkout):
 *   - SimdGemm.SgemmDirect / SgemmDirectParallelM: the no-pack 6x16 kernel that per-head attention GEMMs and thin-M
 *     products take (src/AiDotNet.Tensors/Engines/Simd/SimdGemm.cs:1888-2075 driver, :2792-2866 DirectKernel6x16,
 *     :2987-3041 DirectKernel6x16Store, masked edges :2887-2980, :3048-3140; dispatch gate :1555-1613, thresholds :1725-1767; also reached from BlasManaged.TryThinMDirect,
 *     src/AiDotNet.Tensors/Engines/BlasManaged/BlasManaged.cs:139-215).
 *     Per C element: ONE fused multiply-add chain over the whole of k in ascending order starting from 0, then a plain
 *     store (cleared output) or C + acc (accumulate).  The M-parallel form splits rows among workers and changes no value.
 *   - GotoGemmFp32.RunParallel / RunTile: what large fp32 GEMMs run on hosts with many threads
 *     (src/AiDotNet.Tensors/Engines/BlasManaged/GotoGemmFp32.cs:319-347 tile grid, :421-480 tile, :834-862 scalar tails,
 *     :210-216 tail zeroing, :91-121 block choice).  Per tile and K-panel of kc: 6x16 register tiles run a fused chain from 0
 *     and overwrite C (first panel) or add to it (later panels); rows past the last whole 6 and columns past the last whole 16
 *     of a tile are computed by scalar loops that round the product and the sum separately and add into a zeroed C.
 *   - Simd.FusedAttention.FlashAttentionForward[Ptr] / BatchedFlashAttention: the tiled online-softmax path of compiled plans
 *     (src/AiDotNet.Tensors/Engines/Simd/FusedAttention.cs:39-90 driver, :93-155 scores, :158-235 online softmax, :237-290
 *     helpers) with FastExp256 (src/AiDotNet.Tensors/Engines/Simd/SimdKernels.cs:3025-3077): 32 x 32 tiles, scores = dot * scale
 *     with the dot product's 4 x 8-lane accumulation order, clamp of the exponent argument to [-87.3365, 88.7228] (a masked
 *     logit contributes exp(-87.3365) ~ 1.2e-38, not 0), rescale only when 0 < factor < 1, normalise at the end, no LSE.
 *
 * Pinned by tests/test_oracle_paths.py: dyadic inputs (every order exact: equality with integer arithmetic), exact-rational
 * evaluation of single elements (the fused chain; the separately rounded scalar tails), bit-equality of the direct kernel with
 * the independently written tiled restatement for k <= 512, float64 truth at the reference tests' shapes and bounds
 * (tests/AiDotNet.Tensors.Tests/Engines/BlasManagedThinMDirectTests.cs:27-52, Engines/Compilation/CompilationComponentTests.cs:
 * 110-150), the block-choice table of the source comments, closed forms of the fast exponential (exp(0) = 1, clamp, relative
 * error <= 2e-6 against libm), and agreement of the tiled attention with the float64 softmax.
 * Parity unpinned (stated, inside tolerance): MathF.Exp's last ulp in the rescale factor and the scalar column tail; the
 * JIT-emitted machine-code micro-kernel's instruction order inside a 6x16 tile (assumed: one fused chain per element in k order).
 */
#include <immintrin.h>
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ SgemmDirect */
/* 1 when SgemmAddInternal sends a non-transposed product to the direct kernel (SimdGemm.cs:1575-1613). */
int orc_sgemm_direct_applies(int m, int k, int n)
{
    const long long work = (long long)m * k * n;
    if (m < 6 || n <= 0) return 0;
    const int tall_thin = n >= 16 && n % 8 == 0 && m >= 256 && k <= 512 && work <= 4LL * 1024 * 1024 * 1024;
    return n >= 16 && (work <= 32LL * 1024 * 1024 || tall_thin) && (k <= 512 || tall_thin) && n % 8 == 0;
}

/* 1 when BlasManaged.Gemm<float> takes its thin-M carve-out to the same kernel (contiguous operands, ldc == n;
 * src/AiDotNet.Tensors/Engines/BlasManaged/BlasManaged.cs:116-124 limits, :139-154 gate). */
int orc_thin_m_direct_applies(int m, int n, int k)
{
    if ((n & 7) != 0) return 0;
    if (m < 64 || m > 1024 || n > 512 || k > 1024) return 0;
    return (long long)m * n * k >= (1LL << 20);
}

void orc_sgemm_direct(const float* a, int lda, const float* b, int ldb, float* c, int m, int k, int n, int cleared, int threads)
{
    (void)threads;
#ifdef _OPENMP
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(static)
#endif
    for (int i = 0; i < m; i++) {
        for (int j = 0; j < n; j++) {
            float acc = 0.0f;
            for (int p = 0; p < k; p++) acc = fmaf(a[(long)i * lda + p], b[(long)p * ldb + j], acc);
            c[(long)i * n + j] = cleared ? acc : c[(long)i * n + j] + acc;
        }
    }
}

/* ------------------------------------------------------------------ GotoGemmFp32 */
/* (mc, nc, kc) of GotoGemmFp32.ChooseParallelBlocks(m, n) for a host with `cores` workers (GotoGemmFp32.cs:91-121). */
void orc_goto_choose_blocks(int m, int n, int cores, int* out3)
{
    const int kc = 256;
    if (m >= 1536 && n >= 1536) { out3[0] = 192; out3[1] = 256; out3[2] = kc; return; }
    if (m >= 640 && n >= 640) { out3[0] = 96; out3[1] = 128; out3[2] = kc; return; }
    if (m <= 512) {
        int ic = (int)nearbyint(m / 128.0);          /* Math.Round: ties to even, the default mode of nearbyint */
        if (ic < 1) ic = 1;
        const int mc = (m + ic - 1) / ic;
        int target_jc = (cores + ic - 1) / ic;
        if (target_jc < 1) target_jc = 1;
        int nc = n / target_jc;
        if (nc > 128) nc = 128;
        if (nc < 32) nc = 32;
        nc = (nc / 16) * 16;
        if (nc < 16) nc = 16;
        out3[0] = mc; out3[1] = nc; out3[2] = kc;
        return;
    }
    out3[0] = 120; out3[1] = 128; out3[2] = kc;
}

void orc_goto_gemm(const float* a, int lda, const float* b, int ldb, float* c, int ldc, int m, int n, int k,
                   int mc, int nc, int kc, int threads)
{
    (void)threads;
    if (k <= 0) { for (int i = 0; i < m; i++) for (int j = 0; j < n; j++) c[(long)i * ldc + j] = 0.0f; return; }
    const int num_ic = (m + mc - 1) / mc, num_jc = (n + nc - 1) / nc;
#ifdef _OPENMP
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(dynamic)
#endif
    for (int tile = 0; tile < num_ic * num_jc; tile++) {
        const int ic = (tile % num_ic) * mc, jc = (tile / num_ic) * nc;
        const int eff_mc = m - ic < mc ? m - ic : mc, eff_nc = n - jc < nc ? n - jc : nc;
        const int n_full = eff_nc - eff_nc % 16, m_full = eff_mc - eff_mc % 6;
        for (int pc = 0; pc < k; pc += kc) {
            const int eff_kc = k - pc < kc ? k - pc : kc;
            if (pc == 0) {
                /* ZeroTailStrips: rows past the whole 6-row blocks, and the tail columns of the whole rows */
                for (int r = m_full; r < eff_mc; r++) for (int col = 0; col < eff_nc; col++) c[(long)(ic + r) * ldc + jc + col] = 0.0f;
                for (int r = 0; r < m_full; r++) for (int col = n_full; col < eff_nc; col++) c[(long)(ic + r) * ldc + jc + col] = 0.0f;
            }
            /* whole 6 x 16 register tiles: fused chain from 0 over the panel, overwrite on the first panel, add afterwards */
            for (int r = 0; r < m_full; r++) {
                for (int col = 0; col < n_full; col++) {
                    float acc = 0.0f;
                    for (int kk = 0; kk < eff_kc; kk++) acc = fmaf(a[(long)(ic + r) * lda + pc + kk], b[(long)(pc + kk) * ldb + jc + col], acc);
                    float* dst = c + (long)(ic + r) * ldc + jc + col;
                    *dst = pc == 0 ? acc : *dst + acc;
                }
            }
            /* ScalarTails: product and sum rounded separately (plain C# float arithmetic), added into C */
            for (int r = 0; r < eff_mc; r++) {
                for (int col = n_full; col < eff_nc; col++) {
                    volatile float s = 0.0f;
                    for (int kk = 0; kk < eff_kc; kk++) { volatile float p = a[(long)(ic + r) * lda + pc + kk] * b[(long)(pc + kk) * ldb + jc + col]; s = s + p; }
                    c[(long)(ic + r) * ldc + jc + col] += s;
                }
            }
            for (int r = m_full; r < eff_mc; r++) {
                for (int col = 0; col < n_full; col++) {
                    volatile float s = 0.0f;
                    for (int kk = 0; kk < eff_kc; kk++) { volatile float p = a[(long)(ic + r) * lda + pc + kk] * b[(long)(pc + kk) * ldb + jc + col]; s = s + p; }
                    c[(long)(ic + r) * ldc + jc + col] += s;
                }
            }
        }
    }
}

/* ------------------------------------------------------------------ FastExp256, one lane (SimdKernels.cs:3025-3077) */
float orc_fast_exp(float x)
{
    /* Avx.Max(clampMin, Avx.Min(clampMax, x)): MINPS / MAXPS return the SECOND operand when either is NaN */
    float t = (88.7228f < x) ? 88.7228f : x;          /* min(clampMax, x); NaN compares false -> x */
    x = (-87.3365f > t) ? -87.3365f : t;              /* max(clampMin, t) */
    const float log2e = 1.44269504088896341f, ln2hi = 0.693359375f, ln2lo = -2.12194440e-4f;
    const float n = nearbyintf(x * log2e);            /* round to nearest even */
    float r = fmaf(-n, ln2hi, x);
    r = fmaf(-n, ln2lo, r);
    const float r2 = r * r;
    const float c2 = 0.5f, c3 = 0.166666666666f, c4 = 0.041666666666f, c5 = 0.008333333333f, c6 = 0.001388888888f;
    const float p01 = fmaf(1.0f, r, 1.0f);
    const float p23 = fmaf(c3, r, c2);
    const float p45 = fmaf(c5, r, c4);
    const float r4 = r2 * r2;
    const float lo = fmaf(p23, r2, p01);
    const float hi = fmaf(c6, r2, p45);
    const float poly = fmaf(hi, r4, lo);
    const int32_t ni = (int32_t)n;                    /* exact: n is integral and small */
    const uint32_t bits = (uint32_t)(ni + 127) << 23;
    float scale;
    memcpy(&scale, &bits, 4);
    return poly * scale;
}

/* HorizontalSum of eight lanes (SimdKernels.cs:6424-6480): fold the upper half onto the lower, then (s0 + s1) + (s2 + s3) */
static float hsum8(const float* v)
{
    const float s0 = v[0] + v[4], s1 = v[1] + v[5], s2 = v[2] + v[6], s3 = v[3] + v[7];
    return (s0 + s1) + (s2 + s3);
}

/* DotProductSimd (FusedAttention.cs:112-155) */
static float dot_simd(const float* a, const float* b, int length)
{
    float sum = 0.0f;
    int i = 0;
    if (length >= 32) {
        float acc[4][8];
        memset(acc, 0, sizeof acc);
        const int simd = length & ~31;
        for (; i < simd; i += 32)
            for (int q = 0; q < 4; q++)
                for (int l = 0; l < 8; l++) acc[q][l] = fmaf(a[i + 8 * q + l], b[i + 8 * q + l], acc[q][l]);
        float t[8];
        for (int l = 0; l < 8; l++) t[l] = (acc[0][l] + acc[1][l]) + (acc[2][l] + acc[3][l]);
        sum = hsum8(t);
    } else if (length >= 8) {
        float acc[8] = {0};
        const int simd = length & ~7;
        for (; i < simd; i += 8)
            for (int l = 0; l < 8; l++) acc[l] = fmaf(a[i + l], b[i + l], acc[l]);
        sum = hsum8(acc);
    }
    for (; i < length; i++) { volatile float p = a[i] * b[i]; sum = sum + p; }
    return sum;
}

/* FlashAttentionForwardPtr for one (batch, head): q [seqQ, d], k and v [seqK, d], out [seqQ, d] */
static void fused_attention_one(const float* q, const float* k, const float* v, float* out, int seqQ, int seqK, int d, float scale, int causal)
{
    const int br = seqQ < 32 ? seqQ : 32, bc = seqK < 32 ? seqK : 32;
    float* scores = (float*)malloc(sizeof(float) * (size_t)br * bc);
    float row_max[32], row_sum[32];
    for (long i = 0; i < (long)seqQ * d; i++) out[i] = 0.0f;
    for (int qi = 0; qi < seqQ; qi += br) {
        const int abr = seqQ - qi < br ? seqQ - qi : br;
        for (int r = 0; r < abr; r++) { row_max[r] = -INFINITY; row_sum[r] = 0.0f; }
        for (int kj = 0; kj < seqK; kj += bc) {
            const int abc = seqK - kj < bc ? seqK - kj : bc;
            for (int r = 0; r < abr; r++)
                for (int c = 0; c < abc; c++) scores[r * abc + c] = dot_simd(q + (long)(qi + r) * d, k + (long)(kj + c) * d, d) * scale;
            if (causal)
                for (int r = 0; r < abr; r++)
                    for (int c = 0; c < abc; c++) if (qi + r < kj + c) scores[r * abc + c] = -INFINITY;
            for (int r = 0; r < abr; r++) {
                float* srow = scores + r * abc;
                float* orow = out + (long)(qi + r) * d;
                float local_max = -INFINITY;
                for (int c = 0; c < abc; c++) if (srow[c] > local_max) local_max = srow[c];
                const float prev = row_max[r];
                const float new_max = prev > local_max ? prev : local_max;      /* Math.Max */
                row_max[r] = new_max;
                const float rescale = prev == -INFINITY ? 0.0f : expf(prev - new_max);
                if (rescale > 0.0f && rescale < 1.0f) {
                    for (int i = 0; i < d; i++) orow[i] *= rescale;
                    row_sum[r] *= rescale;
                }
                float local_sum = 0.0f;
                int c = 0;
                if (abc >= 8) {
                    float vsum[8] = {0};
                    const int simd = abc & ~7;
                    for (; c < simd; c += 8)
                        for (int l = 0; l < 8; l++) { const float e = orc_fast_exp(srow[c + l] - new_max); srow[c + l] = e; vsum[l] += e; }
                    local_sum = hsum8(vsum);
                }
                for (; c < abc; c++) { const float e = expf(srow[c] - new_max); srow[c] = e; local_sum += e; }
                for (c = 0; c < abc; c++) {
                    const float w = srow[c];
                    const float* vrow = v + (long)(kj + c) * d;
                    int i = 0;
                    if (d >= 8) for (; i < (d & ~7); i++) orow[i] = fmaf(w, vrow[i], orow[i]);
                    for (; i < d; i++) { volatile float p = w * vrow[i]; orow[i] = orow[i] + p; }
                }
                row_sum[r] += local_sum;
            }
        }
        for (int r = 0; r < abr; r++) {
            const float inv = row_sum[r] > 0.0f ? 1.0f / row_sum[r] : 0.0f;
            float* orow = out + (long)(qi + r) * d;
            for (int i = 0; i < d; i++) orow[i] *= inv;
        }
    }
    free(scores);
}

/* BatchedFlashAttention: q [bh, seqQ, d], k and v [bh, seqK, d] (FusedAttention.cs:292-325) */
void orc_fused_attention_fastexp(const float* q, const float* k, const float* v, float* out, int batch_heads, int seqQ, int seqK, int d,
                                 float scale, int causal, int threads)
{
    (void)threads;
#ifdef _OPENMP
#pragma omp parallel for num_threads(threads > 0 ? threads : 1) schedule(dynamic)
#endif
    for (int bh = 0; bh < batch_heads; bh++)
        fused_attention_one(q + (long)bh * seqQ * d, k + (long)bh * seqK * d, v + (long)bh * seqK * d, out + (long)bh * seqQ * d,
                            seqQ, seqK, d, scale, causal);
}
