/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement ("oracle") of the reference's fused
 * scaled-dot-product attention.  Nothing in the shipped library links, loads or
 * calls this file; only tests, the smoke check and the bench's cpu_baseline leg do.
 *
 * What it restates (paths relative to the reference checkout):
 *   - `CpuEngine.FlashAttentionFloat`: per (batch, head) explicit K^T, S = Q*K^T by
 *     the sequential CPU GEMM, scale (+ bias), causal mask, stable softmax with
 *     expf, LSE = max + log(sum), fully masked row -> zeros and LSE = -inf,
 *     O = P*V by the sequential CPU GEMM
 *     (src/AiDotNet.Tensors/Engines/CpuEngine.cs:29146-29288);
 *   - `CpuEngine.ScaledDotProductAttentionFloat`: same three steps with a boolean
 *     keep-mask broadcast over size-1 axes and the optional tanh soft-cap
 *     (src/AiDotNet.Tensors/Engines/CpuEngine.cs:27695-27881);
 *   - the causal alignment offset `key j masked iff j > i + queryOffset`
 *     (src/AiDotNet.Tensors/Engines/Autodiff/FlashAttention2.cs:58-60, 123, 144-145):
 *     offset 0 is the top-left rule of FlashAttentionFloat (CpuEngine.cs:29235),
 *     offset Sk - Sq is the bottom-right rule of the backend's SDPA kernel
 *     (src/AiDotNet.Tensors/Engines/DirectGpu/HIP/Kernels/HipAttentionKernels.cs:69-71);
 *   - grouped-query head sharing kvHead = h / (heads / kvHeads)
 *     (HipAttentionKernels.cs:60-66);
 *   - the single-query decode loop of the reference's decode test
 *     (tests/AiDotNet.Tensors.Tests/Engines/DirectGpu/FlashDecodeHipTests.cs:43-69).
 *
 * Pinned by (tests/test_oracle_attention.py): an independent fp64 numpy softmax
 * attention; rows of P sum to 1; causal row 0 returns V[0]; Q = 0 returns running
 * means of V; key permutation invariance; LSE against scipy logsumexp; the identity
 * Q/K/V bias case; the soft-cap closed form; decode == last row of causal prefill;
 * all-masked rows.  Parity unpinned (stated, inside tolerance): last-ulp behaviour
 * of the C# MathF.Exp / MathF.Log versus libm expf / logf.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>

void orc_sgemm(const float* a, const float* b, float* c, int m, int k, int n, int threads);

/* Strides are in elements; the head dimension is unit stride. */
typedef struct { long b, h, s; } orc_stride3;

/*
 * q [B,H,Sq,D], k/v [B,Hkv,Sk,D], out [B,H,Sq,D] dense row-major,
 * lse [B,H,Sq] or NULL, weights [B,H,Sq,Sk] or NULL.
 * bias: additive fp32 [B,H,Sq,Sk] (bias_batch_stride = H*Sq*Sk) or [H,Sq,Sk]
 *       (bias_batch_stride = 0) or NULL; added after the scale (CpuEngine.cs:29226-29232).
 * keep: boolean keep-mask bytes or NULL, logical shape keep_shape[4] broadcast over
 *       size-1 axes to [B,H,Sq,Sk]; 0 = masked (CpuEngine.cs:27745-27752, 27808).
 * softcap > 0: v = cap * tanh(v / cap) on the scaled logit, before masking
 *       (CpuEngine.cs:27806-27807).
 * causal != 0: key j is masked iff j > i + query_offset.
 */
void orc_attention_f32(const float* q, const float* k, const float* v,
                       const float* bias, long bias_batch_stride,
                       const uint8_t* keep, const int* keep_shape,
                       float* out, float* lse, float* weights,
                       int B, int H, int Hkv, int Sq, int Sk, int D,
                       float scale, int causal, int query_offset, float softcap, int threads)
{
    if (Hkv <= 0) Hkv = H;
    int group = H / Hkv;
    if (threads < 1) threads = 1;
    #pragma omp parallel for schedule(dynamic, 1) num_threads(threads) if (threads > 1)
    for (int bh = 0; bh < B * H; bh++) {
        int b = bh / H, h = bh % H;
        int kvh = h / group;
        const float* qh = q + (long)bh * Sq * D;
        const float* kh = k + ((long)b * Hkv + kvh) * Sk * D;
        const float* vh = v + ((long)b * Hkv + kvh) * Sk * D;
        float* kt = (float*)malloc((size_t)D * Sk * sizeof(float));
        float* scores = (float*)malloc((size_t)Sq * Sk * sizeof(float));
        float* w = weights ? weights + (long)bh * Sq * Sk : (float*)malloc((size_t)Sq * Sk * sizeof(float));
        for (int i = 0; i < Sk; i++)
            for (int j = 0; j < D; j++) kt[(long)j * Sk + i] = kh[(long)i * D + j];
        orc_sgemm(qh, kt, scores, Sq, D, Sk, 1);

        int mB = 1, mH = 1, mQ = 1, mK = 1;
        if (keep) { mB = keep_shape[0]; mH = keep_shape[1]; mQ = keep_shape[2]; mK = keep_shape[3]; }
        int mb = mB == 1 ? 0 : b, mh = mH == 1 ? 0 : h;
        float inv_cap = softcap > 0.0f ? 1.0f / softcap : 0.0f;

        for (int i = 0; i < Sq; i++) {
            float* srow = scores + (long)i * Sk;
            float* wrow = w + (long)i * Sk;
            float maxv = -INFINITY;
            for (int j = 0; j < Sk; j++) {
                float x = srow[j] * scale;
                if (softcap > 0.0f) x = softcap * tanhf(x * inv_cap);
                if (bias) x += bias[(long)b * bias_batch_stride + (long)h * Sq * Sk + (long)i * Sk + j];
                if (keep) {
                    int mi = mQ == 1 ? 0 : i, mj = mK == 1 ? 0 : j;
                    if (!keep[(((long)mb * mH + mh) * mQ + mi) * mK + mj]) x = -INFINITY;
                }
                if (causal && j > i + query_offset) x = -INFINITY;
                if (x > maxv) maxv = x;
                srow[j] = x;
            }
            if (isinf(maxv) && maxv < 0) {
                for (int j = 0; j < Sk; j++) wrow[j] = 0.0f;
                if (lse) lse[(long)bh * Sq + i] = -INFINITY;
                continue;
            }
            float sum = 0.0f;
            for (int j = 0; j < Sk; j++) { float e = expf(srow[j] - maxv); wrow[j] = e; sum += e; }
            float inv = sum != 0.0f ? 1.0f / sum : 0.0f;
            for (int j = 0; j < Sk; j++) wrow[j] *= inv;
            if (lse) lse[(long)bh * Sq + i] = maxv + logf(sum);
        }
        orc_sgemm(w, vh, out + (long)bh * Sq * D, Sq, Sk, D, 1);
        free(kt); free(scores);
        if (!weights) free(w);
    }
}

/* fp64 truth of the same definition (inputs are float, every intermediate double). */
void orc_attention_f64(const float* q, const float* k, const float* v,
                       const float* bias, long bias_batch_stride,
                       const uint8_t* keep, const int* keep_shape,
                       double* out, double* lse,
                       int B, int H, int Hkv, int Sq, int Sk, int D,
                       double scale, int causal, int query_offset, double softcap, int threads)
{
    if (Hkv <= 0) Hkv = H;
    int group = H / Hkv;
    if (threads < 1) threads = 1;
    #pragma omp parallel for schedule(dynamic, 1) num_threads(threads) if (threads > 1)
    for (int bh = 0; bh < B * H; bh++) {
        int b = bh / H, h = bh % H;
        int kvh = h / group;
        const float* qh = q + (long)bh * Sq * D;
        const float* kh = k + ((long)b * Hkv + kvh) * Sk * D;
        const float* vh = v + ((long)b * Hkv + kvh) * Sk * D;
        double* p = (double*)malloc((size_t)Sk * sizeof(double));
        int mB = 1, mH = 1, mQ = 1, mK = 1;
        if (keep) { mB = keep_shape[0]; mH = keep_shape[1]; mQ = keep_shape[2]; mK = keep_shape[3]; }
        int mb = mB == 1 ? 0 : b, mh = mH == 1 ? 0 : h;
        for (int i = 0; i < Sq; i++) {
            double maxv = -INFINITY;
            for (int j = 0; j < Sk; j++) {
                double s = 0.0;
                for (int d = 0; d < D; d++) s += (double)qh[(long)i * D + d] * (double)kh[(long)j * D + d];
                double x = s * scale;
                if (softcap > 0.0) x = softcap * tanh(x / softcap);
                if (bias) x += (double)bias[(long)b * bias_batch_stride + (long)h * Sq * Sk + (long)i * Sk + j];
                if (keep) {
                    int mi = mQ == 1 ? 0 : i, mj = mK == 1 ? 0 : j;
                    if (!keep[(((long)mb * mH + mh) * mQ + mi) * mK + mj]) x = -INFINITY;
                }
                if (causal && j > i + query_offset) x = -INFINITY;
                if (x > maxv) maxv = x;
                p[j] = x;
            }
            double* orow = out + ((long)bh * Sq + i) * D;
            for (int d = 0; d < D; d++) orow[d] = 0.0;
            if (isinf(maxv) && maxv < 0) { if (lse) lse[(long)bh * Sq + i] = -INFINITY; continue; }
            double sum = 0.0;
            for (int j = 0; j < Sk; j++) { p[j] = exp(p[j] - maxv); sum += p[j]; }
            for (int j = 0; j < Sk; j++) {
                double wj = p[j] / sum;
                if (wj == 0.0) continue;
                for (int d = 0; d < D; d++) orow[d] += wj * (double)vh[(long)j * D + d];
            }
            if (lse) lse[(long)bh * Sq + i] = maxv + log(sum);
        }
        free(p);
    }
}

/* Single-query decode of one sequence over K/V laid out [seqLen, kvHeads, headDim]:
 * logits, max, exp, denominator, then out += (e / denom) * v, all fp32 in key order.
 * FlashDecodeHipTests.cs:43-69 (DecodeOracle).  q and out are [heads, headDim]. */
void orc_decode_f32(const float* q, const float* k, const float* v, float* out,
                    int heads, int kvHeads, int headDim, int seqLen, float scale)
{
    float* logits = (float*)malloc((size_t)seqLen * sizeof(float));
    for (int h = 0; h < heads; h++) {
        int kvh = h / (heads / kvHeads);
        float maxv = -INFINITY;
        for (int t = 0; t < seqLen; t++) {
            const float* kr = k + ((long)t * kvHeads + kvh) * headDim;
            float dot = 0.0f;
            for (int d = 0; d < headDim; d++) dot += q[(long)h * headDim + d] * kr[d];
            logits[t] = dot * scale;
            if (logits[t] > maxv) maxv = logits[t];
        }
        float denom = 0.0f;
        for (int t = 0; t < seqLen; t++) { logits[t] = expf(logits[t] - maxv); denom += logits[t]; }
        float* o = out + (long)h * headDim;
        for (int d = 0; d < headDim; d++) o[d] = 0.0f;
        for (int t = 0; t < seqLen; t++) {
            const float* vr = v + ((long)t * kvHeads + kvh) * headDim;
            float p = logits[t] / denom;
            for (int d = 0; d < headDim; d++) o[d] += p * vr[d];
        }
    }
    free(logits);
}
