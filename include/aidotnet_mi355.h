/*
 * aidotnet_mi355.h -- C ABI of libaidotnet_mi355.so: hand-written gfx950 (MI355X) kernels for the
 * GEMM and fused-attention members of AiDotNet.Tensors' GPU-backend slot.
 *
 * These are the entry points a P/Invoke binding in the reference's HIP backend would bind in
 * place of its hipBLAS calls and run-time compiled kernel strings.  Paths below are relative to
 * the reference checkout (src/AiDotNet.Tensors/...).
 *
 * Conventions (mirroring Engines/DirectGpu/HIP/HipNativeBindings.cs:13-87, 342-641 and
 * HipBlasNative.cs:16-27, 82-157): cdecl, blittable arguments only, every function returns an int
 * status (0 = success); all pointers are raw device pointers (IGpuBuffer.Handle,
 * Engines/DirectGpu/IDirectGpuBackend.cs:3776-3803) owned by the caller and never retained;
 * matrices are dense row-major; `stream` is a hipStream_t (NULL = the default stream).  Work is
 * enqueued on `stream` and the call returns without waiting: a caller that keeps the reference's
 * "result ready on return" contract (HipBackend.cs:1444-1446) calls aidn_mi355_sync afterwards.
 * fp16 / bf16 values travel as raw 16-bit patterns (uint16_t).  Every output element is
 * overwritten (pooled buffers may hold stale data; beta == 0 never reads C).
 */
#ifndef AIDOTNET_MI355_H
#define AIDOTNET_MI355_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Exported with default visibility; everything else in the library is hidden. */
#if defined(__GNUC__)
#define AIDN_API __attribute__((visibility("default")))
#else
#define AIDN_API
#endif

/* Status codes. Values 1000+ are this library's; any other non-zero value is a hipError_t. */
enum {
    AIDN_OK = 0,
    AIDN_ERR_INVALID_ARGUMENT = 1001,   /* null pointer, non-positive dimension, bad ratio */
    AIDN_ERR_UNSUPPORTED = 1002,        /* e.g. head dimension the kernels do not cover */
    AIDN_ERR_NO_DEVICE = 1003,          /* no gfx950 device */
    AIDN_ERR_OUT_OF_MEMORY = 1004,      /* library-owned workspace could not be allocated */
    AIDN_ERR_WORKSPACE = 1005           /* the workspace would have to grow while the stream is being captured */
};

/* ---- lifetime ------------------------------------------------------------------------------
 * One context per backend instance (the reference creates one stream + one hipBLAS handle per
 * HipBackend, HipBackend.cs:246, 288, 371).  The context owns only the library's private
 * workspace (split-KV and split-K partials, intermediates of the fused MHA forward), one per stream
 * the context has been called on, so calls on different streams never share it; it grows on demand
 * (a block that has been handed to a kernel is never freed before aidn_mi355_destroy, so queued work
 * and captured graphs keep valid addresses) and is released by aidn_mi355_destroy.  Calls on the SAME
 * stream run in order and may share it.  The context may be used from several host threads; every call
 * must be made with the context's device current on the calling thread (hipSetDevice(device) -- the
 * library launches on the caller's current device and does not switch it: aidn_mi355_create leaves
 * `device` current on the thread that called it, other threads set it themselves; the reference's
 * backend likewise selects its device once, in its constructor, HipBackend.cs:246). */
AIDN_API int aidn_mi355_create(int device, void** ctx);
AIDN_API int aidn_mi355_destroy(void* ctx);
/* Text of the last failure on this context (never NULL; empty when none). */
AIDN_API const char* aidn_mi355_last_error(void* ctx);
AIDN_API const char* aidn_mi355_version(void);
/* hipStreamSynchronize(stream): replaces HipBackend.Synchronize (HipBackend.cs:1444-1446). */
AIDN_API int aidn_mi355_sync(void* ctx, void* stream);
/* Makes the workspace of `stream` at least `bytes` large now, so that later calls on it allocate nothing -- required before
 * the calls are captured into a HIP graph (no allocation can happen during capture: a decode or fused-MHA call, which cannot
 * run without its workspace, then returns AIDN_ERR_WORKSPACE; a GEMM or prefill-attention call takes its kernel that needs none);
 * one eager run of the same call sequence has the same effect.  aidn_mi355_workspace_bytes reads the current size (after a
 * warm-up run: the amount to reserve on another stream or context).  No counterpart in the reference, whose backend allocates
 * per call from its buffer pool (HipBackend.cs:12214-12270). */
AIDN_API int aidn_mi355_reserve_workspace(void* ctx, void* stream, uint64_t bytes);
AIDN_API uint64_t aidn_mi355_workspace_bytes(void* ctx, void* stream);
/* Gives back the workspace the context holds for `stream` (waits for the stream first, then frees the current block and every
 * block retired by growth): for callers that create and destroy streams, since a block is otherwise kept until
 * aidn_mi355_destroy.  Graphs captured from this stream must not be replayed afterwards (they hold the freed addresses).
 * AIDN_ERR_WORKSPACE while the stream is being captured.  No counterpart in the reference (its buffers return to a pool per
 * call, HipBackend.cs:12214-12270). */
AIDN_API int aidn_mi355_release_stream_workspace(void* ctx, void* stream);

/* ---- fp32 GEMM -------------------------------------------------------------------------------
 * C[M,N] = alpha * A[M,K] * op(B) + beta * C.  transB == 0: B is [K,N]; transB != 0: B is stored
 * [N,K] (C = A * B^T).  Replaces IDirectGpuBackend.Gemm (IDirectGpuBackend.cs:160-172; host
 * HipBackend.cs:1370-1447, hipblasSgemm :1502-1545) and MatMulTransposed (:184-203; host
 * HipBackend.cs:1450-1490).  Argument order (M, N, K) as at that layer.  True fp32 MFMA, fp32
 * accumulation (no TF32-style truncation).  M <= 8 with B [K,N] takes the bandwidth-bound small-M path (B streamed once,
 * split-K partials in the context workspace, summed in a fixed order): the GPU form of SimdGemm.SgemmNParallelSmallM /
 * SgemmConcatenatedProjections (Engines/Simd/SimdGemm.NParallelSmallM.cs:31-109); the same holds for the bias/activation
 * and fp16-weight entry points below.  With 9 <= M <= 32 (B [K,N], N a multiple of 128, K a multiple of 32) the weight matrix is
 * likewise streamed once, through a 32-row MFMA kernel, and larger products whose tiles would not fill the chip over a long K
 * (K >= 1024, K a multiple of 32, either layout of B) run their K ranges side by side; both keep fp32 partials in the context
 * workspace and sum them in range order, so results are repeatable run to run (this entry point and the bias/activation one).
 * Rows that are not whole 16-byte chunks (K, or N with B [K,N], not a multiple of 4): a product of some size is computed from
 * zero-padded copies of A and B in the workspace (same sums; C is written in place). */
AIDN_API int aidn_mi355_sgemm(void* ctx, void* stream, const float* A, const float* B, float* C,
                     int M, int N, int K, float alpha, float beta, int transB);

/* batch independent products on concatenated matrices: A[i] is M x K at A + i*M*K, B[i] K x N,
 * C[i] M x N.  Replaces IDirectGpuBackend.BatchedGemm (IDirectGpuBackend.cs:205-222; host
 * HipBackend.cs:1599-1631). */
AIDN_API int aidn_mi355_sgemm_batched(void* ctx, void* stream, const float* A, const float* B, float* C,
                             int M, int N, int K, int batch, float alpha, float beta);

/* ---- fused projection epilogues ---------------------------------------------------------------
 * C[M,N] = act(A[M,K] * B[K,N] + bias[N]), bias broadcast over rows (may be null), in one kernel.
 * activation: 0 none, 1 ReLU, 2 GELU (tanh form), 3 sigmoid, 4 tanh, 5 leaky ReLU with slope act_param,
 * 6 swish -- the numbering of FusedActivationType (Engines/FusedActivationType.cs:23-70).  Replaces
 * IDirectGpuBackend.GemmBias / GemmBiasRelu / GemmBiasGelu / GemmBiasSigmoid / GemmBiasTanh /
 * GemmBiasSwish / GemmBiasLeakyRelu (IDirectGpuBackend.cs:227-275; host HipBackend.cs:1637-1785, which
 * runs the GEMM, a bias kernel and an activation kernel one after the other) and is what
 * IEngine.FusedLinear needs (Engines/IEngine.cs:5166; CPU epilogue Helpers/CpuFusedOperations.cs:590-700).
 * The 16-bit forms take fp16 / bf16 A and B, an fp32 bias, accumulate and apply the epilogue in fp32 and
 * store fp32 (out_is_f32 != 0) or one rounding to the input type. */
AIDN_API int aidn_mi355_sgemm_bias_act(void* ctx, void* stream, const float* A, const float* B, const float* bias, float* C,
                              int M, int N, int K, int activation, float act_param);
AIDN_API int aidn_mi355_hgemm_bias_act(void* ctx, void* stream, const uint16_t* A, const uint16_t* B, const float* bias, void* C,
                              int out_is_f32, int M, int N, int K, int activation, float act_param);
AIDN_API int aidn_mi355_bf16gemm_bias_act(void* ctx, void* stream, const uint16_t* A, const uint16_t* B, const float* bias, void* C,
                                 int out_is_f32, int M, int N, int K, int activation, float act_param);

/* ---- weight-only fp16 GEMM ----------------------------------------------------------------------
 * C[M,N] = act(A[M,K] * widen(B_f16[K,N]) + bias): fp32 activations, fp16 weights widened exactly on the way into LDS (never
 * materialised in fp32), fp32 products and accumulation, the same optional epilogue as above (bias may be null,
 * activation 0 = none).  The GPU form of SimdGemm.SgemmFp16WeightB / PackBFromHalf
 * (Engines/Simd/SimdGemm.Fp16Weight.cs:22-91, 208-261), reached through CpuEngine.TensorMatMulFp16WeightB and
 * FusedLinearFp16WeightB; the reference has no GPU member for it. */
AIDN_API int aidn_mi355_sgemm_f16weight(void* ctx, void* stream, const float* A, const uint16_t* B_f16, const float* bias, float* C,
                               int M, int N, int K, int activation, float act_param);

/* ---- pre-packed weight operand -----------------------------------------------------------------------
 * The GPU form of the reference's cached packed B (SimdGemm.SgemmWithCachedB and its PrePackedB cache, Engines/Simd/SimdGemm.cs:327-684,
 * 1030-1159: a weight matrix is packed once into the layout the kernel wants and re-used by every later product; results are those of
 * the plain call).  Here the packed layout is the weight zero-padded to whole tiles with 16-byte aligned rows, which is what a product
 * whose N or K is odd (a vocabulary of 50257 columns) otherwise copies on every call.  kind: 0 fp32 (B [K,N], or [N,K] when transB != 0),
 * 1 fp16, 2 bf16 (B [K,N], transB must be 0).  The caller owns `packed` (aidn_mi355_packed_b_bytes bytes, 16-byte aligned) and repacks
 * when the weight changes -- no identity or content check is made here; the reference's cache keys (array identity, version,
 * FNV-1a of the contents) are host-side bookkeeping that stays with the caller.
 * aidn_mi355_gemm_packed_b: C[M,N] = act(A[M,K] * B + bias) with B given in packed form; 16-bit kinds store fp32 (out_is_f32 != 0) or
 * the input type; fp32 ignores out_is_f32.  Same sums as the plain entry points (bit-identical on inputs whose partial sums are exact).
 * Needs the stream's workspace (a padded copy of A when K is not a whole tile, split-K partials): under capture reserve it first. */
AIDN_API uint64_t aidn_mi355_packed_b_bytes(int kind, int K, int N, int transB);
AIDN_API int aidn_mi355_pack_b(void* ctx, void* stream, int kind, const void* B, int K, int N, int transB, void* packed);
AIDN_API int aidn_mi355_gemm_packed_b(void* ctx, void* stream, int kind, const void* A, const void* packedB, const float* bias, void* C,
                             int out_is_f32, int M, int N, int K, int transB, int activation, float act_param);

/* ---- 16-bit GEMM, fp32 accumulation ------------------------------------------------------------
 * C[M,N] = A[M,K] * B[K,N].  *_f32out replaces IGpuHalfPrecisionBackend.GemmFp16In32fOut
 * (Engines/Gpu/IGpuHalfPrecisionBackend.cs:39-48; host HipBackend.HalfPrecision.cs:125-150,
 * hipblasGemmEx); *_f16out replaces Hgemm (:27-37; host :97-122) with fp32 accumulation and one
 * round-to-nearest-even narrow, the arithmetic of the CPU kernel (Engines/Simd/HalfKernels.cs:35-99).
 * The bf16 pair has no member in the reference's backend interface today (its planner widens
 * bf16 tensors to fp32, Engines/Gpu/GpuPrecisionPolicy.cs:497-532); it follows the CPU kernel
 * Engines/Simd/BFloat16Kernels.cs:144-211 and NumericOperations/BFloat16.cs:64-90.
 * Any M, N and K are accepted.  When N or K is not a multiple of 8 (rows that are not whole 16-byte chunks) a product of some size
 * is computed from zero-padded copies of A and B held in the stream's workspace -- same sums, three more passes over the
 * operands; a weight of such a width that is used many times is better stored padded by the caller. */
AIDN_API int aidn_mi355_hgemm_f32out(void* ctx, void* stream, const uint16_t* A, const uint16_t* B, float* C, int M, int N, int K);
AIDN_API int aidn_mi355_hgemm_f16out(void* ctx, void* stream, const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K);
AIDN_API int aidn_mi355_bf16gemm_f32out(void* ctx, void* stream, const uint16_t* A, const uint16_t* B, float* C, int M, int N, int K);
AIDN_API int aidn_mi355_bf16gemm_bf16out(void* ctx, void* stream, const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K);

/* ---- projection + rotary embedding in one call ---------------------------------------------------------
 * C[M,N] = A[M,K] * B[K,N] (fp32 accumulation, C rounded to the inputs' type), then the interleaved rotary embedding of
 * aidn_mi355_rope_interleaved_* over the first rope_cols columns of C: those columns are heads of head_dim elements side by
 * side (the Q and K parts of a concatenated [Wq|Wk|Wv] projection; rope_cols = N rotates everything, a multiple of head_dim), the
 * pair (2i, 2i+1) of a head in row m turns by the angle of position start_position + m % seq_len (rows are [leading, seq_len]:
 * M = batch and seq_len = 1 in a decode step).  The result is what the product followed by the rotation kernel gives, rounding
 * included.  Where the product has a summing pass of its own (few rows: the weight is streamed once in K ranges side by side,
 * the decode-step shapes) the rotation rides on that pass and no separate launch is made; other shapes run the rotation as a
 * second launch over C.  The decode step the reference composes from SimdGemm.SgemmConcatenatedProjections
 * (Engines/Simd/SimdGemm.NParallelSmallM.cs:95-109) and RopeInterleaved (IDirectGpuBackend.cs:1427-1446); no single member of the
 * reference does both. */
AIDN_API int aidn_mi355_hgemm_rope(void* ctx, void* stream, const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K,
                          const float* cos_cache, const float* sin_cache, int head_dim, int rope_cols, int seq_len, int start_position);
AIDN_API int aidn_mi355_bf16gemm_rope(void* ctx, void* stream, const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K,
                             const float* cos_cache, const float* sin_cache, int head_dim, int rope_cols, int seq_len, int start_position);

/* ---- storage conversions ------------------------------------------------------------------------
 * Replace IDirectGpuBackend.ConvertToFp16 / ConvertToFp32 (IDirectGpuBackend.cs:1876-1911; host
 * HipBackend.cs:11942-11981).  n = element count.  Narrowing is round-to-nearest-even; the bf16
 * rule is BFloat16.FromFloat (NumericOperations/BFloat16.cs:64-82), NaN keeps a quiet bit. */
AIDN_API int aidn_mi355_convert_f32_to_f16(void* ctx, void* stream, const float* in, uint16_t* out, int64_t n);
AIDN_API int aidn_mi355_convert_f16_to_f32(void* ctx, void* stream, const uint16_t* in, float* out, int64_t n);
AIDN_API int aidn_mi355_convert_f32_to_bf16(void* ctx, void* stream, const float* in, uint16_t* out, int64_t n);
AIDN_API int aidn_mi355_convert_bf16_to_f32(void* ctx, void* stream, const uint16_t* in, float* out, int64_t n);

/* ---- fused scaled-dot-product attention (forward) -------------------------------------------------
 * O = softmax(scale * Q K^T (+ soft-cap, + bias, masks)) V per (batch, head), computed in tiles with
 * an online softmax: the [Sq,Sk] score matrix is never written unless `weights` is requested.
 *
 * One descriptor covers IDirectGpuBackend.FlashAttentionV2 (IDirectGpuBackend.cs:1451-1471; host
 * HipBackend.cs:6261-6302), FlashAttention (:1448-1449) and ScaledDotProductAttention
 * (:1395-1424; host HipBackend.cs:6118-6175); the value semantics are the CPU engine's
 * (Engines/CpuEngine.cs:29146-29288 and 27695-27881).
 *
 *   q [B,H,Sq,D], k and v [B,Hkv,Sk,D], o [B,H,Sq,D]; the head dimension is unit stride; the
 *   batch / head / row strides are given in ELEMENTS (0 in every stride of a tensor = dense).
 *   H % Hkv == 0; query head h reads kv head h / (H / Hkv)  (HipAttentionKernels.cs:60-66).
 *   lse      [B,H,Sq] fp32 or NULL: max + log(sum) per row (CpuEngine.cs:29262-29263); -inf for a
 *            row with every key masked, whose output row is all zeros (CpuEngine.cs:29243-29249).
 *   causal   != 0: key j is masked iff j > i + causal_query_offset.  Offset 0 is the top-left rule
 *            of FlashAttention / FlashAttentionV2 (CpuEngine.cs:29235, HipAttentionKernels.cs:199);
 *            offset Sk - Sq is the bottom-right rule of ScaledDotProductAttention
 *            (HipAttentionKernels.cs:69-71); same parameter as FlashAttentionConfig.QueryOffset
 *            (Engines/Autodiff/FlashAttention2.cs:58-60, 123, 144-145).
 *   bias     additive fp32 [B,H,Sq,Sk] (bias_batch_stride = H*Sq*Sk) or [H,Sq,Sk]
 *            (bias_batch_stride = 0), added after the scale, or NULL (IDirectGpuBackend.cs:1465-1466).
 *   mask     fp32, 0.0f = masked, anything else = keep (HipAttentionKernels.cs:78); mask_mode 0 none,
 *            1 one [Sq,Sk] plane shared by all (batch, head), 2 full [B,H,Sq,Sk]
 *            (HipBackend.cs:6150-6151).
 *   softcap  > 0: logit = softcap * tanh(scale * qk / softcap) before bias / masks
 *            (CpuEngine.cs:27806-27807); 0 disables.
 *   weights  fp32 [B,H,Sq,Sk] normalised probabilities or NULL (the optional attentionWeights of
 *            ScaledDotProductAttention); written by a second pass from the saved LSE.
 * 16-bit variants: q, k, v are fp16 / bf16 patterns, softmax and accumulation are fp32, the output
 * is fp32 (out_is_16bit == 0; the reference's only reduced-precision attention contract: fp16 in,
 * fp32 O and LSE out, Engines/DirectGpuTensorEngine.cs:11143-11167) or the input type
 * (out_is_16bit != 0).  Any 1 <= D <= 256 is accepted (GpuKernelGuards.MaxHeadDim,
 * Engines/DirectGpu/GpuKernelGuards.cs:12; larger: AIDN_ERR_UNSUPPORTED); rows whose start and strides
 * are multiples of 16 bytes take the vector loads, head dimensions 64 and 128 with such rows the
 * direct-to-LDS kernels.  A 16-bit call at head dimension 128 with few query rows against many keys (chunked prefill, a few
 * speculative tokens) runs the key ranges of a query tile side by side and merges them; the partials live in the stream's
 * workspace (a stream under capture whose workspace would have to grow runs the call unsplit).
 */
typedef struct aidn_attn_desc {
    int32_t B, H, Hkv, Sq, Sk, D;
    float scale;
    int32_t causal;
    int32_t causal_query_offset;
    float softcap;
    int32_t mask_mode;
    int32_t out_is_16bit;
    int64_t bias_batch_stride;
    int64_t q_strides[3];   /* batch, head, row (elements); all zero = dense [B,H,Sq,D] */
    int64_t k_strides[3];
    int64_t v_strides[3];
    int64_t o_strides[3];
} aidn_attn_desc;

AIDN_API int aidn_mi355_attn_fwd_f32(void* ctx, void* stream, const aidn_attn_desc* desc,
                            const float* q, const float* k, const float* v, float* o,
                            float* lse, const float* bias, const float* mask, float* weights);
AIDN_API int aidn_mi355_attn_fwd_f16(void* ctx, void* stream, const aidn_attn_desc* desc,
                            const uint16_t* q, const uint16_t* k, const uint16_t* v, void* o,
                            float* lse, const float* bias, const float* mask, float* weights);
AIDN_API int aidn_mi355_attn_fwd_bf16(void* ctx, void* stream, const aidn_attn_desc* desc,
                             const uint16_t* q, const uint16_t* k, const uint16_t* v, void* o,
                             float* lse, const float* bias, const float* mask, float* weights);

/* ---- decode attention (Sq == 1) ---------------------------------------------------------------------
 * One query row per (batch, head) against a KV cache of Sk rows: HBM-bound, the keys are split over
 * workgroups (coalesced 128-bit loads), partial (max, sum, acc) triples are merged by a second
 * kernel from a library-owned workspace.  Same descriptor (Sq must be 1; with causal != 0 keys
 * j > causal_query_offset are masked, so offset Sk - 1, the bottom-right rule, attends to the whole
 * cache; bias, mask and soft-cap are not available here: a descriptor with softcap > 0 or
 * mask_mode != 0 is refused with AIDN_ERR_UNSUPPORTED -- use aidn_mi355_attn_fwd_* with Sq = 1 for those); strides select the cache
 * layout: [B,Hkv,Sk,D] (dense), the reference's decode layout [Sk,Hkv,D]
 * (HipFlashDecodeKernels.cs:9-10; host FlashDecode HipBackend.cs:919-965) or its dense KVCache
 * [B,Sk,Hkv,D] (Engines/Autodiff/KVCache.cs:5-8).  splits <= 0 picks the split count
 * (the reference default is min(Sk, 8), HipBackend.cs:936); results do not depend on it beyond
 * rounding.  o is fp32 or the input type per desc->out_is_16bit.  Grouped-query caches (Hkv < H) in fp16 / bf16 at head
 * dimension 128 with 16-byte aligned rows fetch each K/V row once for all query heads of its group (the group runs as the rows
 * of one query tile on the matrix cores; the probabilities are rounded to the input type there, as in the prefill kernel). */
AIDN_API int aidn_mi355_attn_decode_f32(void* ctx, void* stream, const aidn_attn_desc* desc,
                               const float* q, const float* k, const float* v, float* o, float* lse, int splits);
AIDN_API int aidn_mi355_attn_decode_f16(void* ctx, void* stream, const aidn_attn_desc* desc,
                               const uint16_t* q, const uint16_t* k, const uint16_t* v, void* o, float* lse, int splits);
AIDN_API int aidn_mi355_attn_decode_bf16(void* ctx, void* stream, const aidn_attn_desc* desc,
                                const uint16_t* q, const uint16_t* k, const uint16_t* v, void* o, float* lse, int splits);
/* aidn_mi355_attn_decode_bf16 for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): same arguments and results, but the split-KV partials live in a static 8 MiB
 * device array of the library instead of the context workspace, so the call never allocates or frees.  Problems whose partials
 * (B * H * splits * (2 + head dimension padded to a power-of-two number of 16-byte chunks) floats) exceed 8 MiB are refused with
 * AIDN_ERR_UNSUPPORTED.  Every call on a GPU shares that GPU's array: calls that overlap in time on one GPU (different
 * streams) race; calls on one stream are ordered.  Nothing in the array has to start at zero.  No counterpart in the
 * reference. */
AIDN_API int aidn_mi355_attn_decode_bf16_noalloc(void* ctx, void* stream, const aidn_attn_desc* desc,
                                        const uint16_t* q, const uint16_t* k, const uint16_t* v, void* o, float* lse, int splits);

/* ---- attention over a paged K/V cache --------------------------------------------------------------------
 * K and V pools [numBlocks, blockSize, kvHeads, headDim]; block_table[i] = pool block of logical block i (int32, at least
 * ceil(keyLen / blockSize) entries); q and o [numQueries, heads, headDim]; o is fp32 for every input type.  kv_heads <= 0
 * means heads.  *_decode: one query over seq_len keys, splits as for aidn_mi355_attn_decode_*.  *_prefill: causal, query i
 * (logical position start_pos + i) sees keys 0 .. start_pos + i.  Replace IDirectGpuBackend.PagedAttentionDecode[Gqa] /
 * PagedAttentionPrefill[Gqa] (IDirectGpuBackend.cs:3614-3633; host HipBackend.cs:831-913, one thread per head in
 * Kernels/HipPagedAttentionKernels.cs:26-58); the reference interface is fp32 only, the 16-bit forms are additions. */
AIDN_API int aidn_mi355_paged_attn_decode_f32(void* ctx, void* stream, const float* q, const float* kcache, const float* vcache,
                                     const int32_t* block_table, float* o, int heads, int kv_heads, int head_dim, int block_size,
                                     int seq_len, float scale, int splits);
AIDN_API int aidn_mi355_paged_attn_decode_f16(void* ctx, void* stream, const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache,
                                     const int32_t* block_table, float* o, int heads, int kv_heads, int head_dim, int block_size,
                                     int seq_len, float scale, int splits);
AIDN_API int aidn_mi355_paged_attn_decode_bf16(void* ctx, void* stream, const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache,
                                      const int32_t* block_table, float* o, int heads, int kv_heads, int head_dim, int block_size,
                                      int seq_len, float scale, int splits);
AIDN_API int aidn_mi355_paged_attn_prefill_f32(void* ctx, void* stream, const float* q, const float* kcache, const float* vcache,
                                      const int32_t* block_table, float* o, int heads, int kv_heads, int head_dim, int block_size,
                                      int num_queries, int start_pos, float scale);
AIDN_API int aidn_mi355_paged_attn_prefill_f16(void* ctx, void* stream, const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache,
                                      const int32_t* block_table, float* o, int heads, int kv_heads, int head_dim, int block_size,
                                      int num_queries, int start_pos, float scale);
AIDN_API int aidn_mi355_paged_attn_prefill_bf16(void* ctx, void* stream, const uint16_t* q, const uint16_t* kcache, const uint16_t* vcache,
                                       const int32_t* block_table, float* o, int heads, int kv_heads, int head_dim, int block_size,
                                       int num_queries, int start_pos, float scale);

/* ---- rotary position embedding, interleaved pairs -----------------------------------------------------------
 * output[r, 2i] = x[r, 2i] cos - x[r, 2i+1] sin, output[r, 2i+1] = x[r, 2i] sin + x[r, 2i+1] cos with the angle of absolute
 * position start_position + r % seq_len; input / output [rows, head_dim] (rows = leading x seq_len), caches fp32
 * [maxSeq, head_dim / 2] with at least start_position + seq_len rows; output may alias input.  Replaces
 * IDirectGpuBackend.RopeInterleaved (IDirectGpuBackend.cs:1427-1446; host HipBackend.cs:6177-6210, kernel
 * Kernels/HipAttentionKernels.cs:958-989).  The 16-bit forms rotate in fp32 and round once. */
AIDN_API int aidn_mi355_rope_interleaved_f32(void* ctx, void* stream, const float* input, const float* cos_cache, const float* sin_cache,
                                    float* output, int64_t rows, int head_dim, int seq_len, int start_position);
AIDN_API int aidn_mi355_rope_interleaved_f16(void* ctx, void* stream, const uint16_t* input, const float* cos_cache, const float* sin_cache,
                                    uint16_t* output, int64_t rows, int head_dim, int seq_len, int start_position);
AIDN_API int aidn_mi355_rope_interleaved_bf16(void* ctx, void* stream, const uint16_t* input, const float* cos_cache, const float* sin_cache,
                                     uint16_t* output, int64_t rows, int head_dim, int seq_len, int start_position);

/* ---- multi-head attention forward --------------------------------------------------------------------
 * output[B,S,dModel] = (softmax(Q K^T / sqrt(d)) V) Wo with [Q|K|V] = input[B,S,dModel] [Wq|Wk|Wv], heads = dModel / d, all
 * weights [dModel,dModel] row-major, no biases: IEngine.MultiHeadAttentionForward (Engines/CpuEngine.MultiHeadAttention.cs:68-143;
 * fp32 path :155-285, fused SDPA over the packed activation :358-522), which has no GPU route in the reference.
 * Three launches and no permutes: one GEMM writes the packed [B*S, 3 dModel] activation, the attention kernel reads it through
 * strides and writes [B,S,H,d], one GEMM projects.  mask (may be null): fp32, non-zero = keep; mask_mode 1 = one [S,S] plane
 * shared by all (b,h), 2 = full [B,H,S,S] (what a broadcast of the reference's Tensor<bool> mask materialises to).
 * The 16-bit forms keep every intermediate in the input type and accumulate in fp32.  Intermediates live in the context's workspace. */
AIDN_API int aidn_mi355_mha_fwd_f32(void* ctx, void* stream, const float* input, const float* wq, const float* wk, const float* wv,
                           const float* wo, const float* mask, int mask_mode, float* output, int B, int S, int dModel, int heads);
AIDN_API int aidn_mi355_mha_fwd_f16(void* ctx, void* stream, const uint16_t* input, const uint16_t* wq, const uint16_t* wk, const uint16_t* wv,
                           const uint16_t* wo, const float* mask, int mask_mode, uint16_t* output, int B, int S, int dModel, int heads);
AIDN_API int aidn_mi355_mha_fwd_bf16(void* ctx, void* stream, const uint16_t* input, const uint16_t* wq, const uint16_t* wk, const uint16_t* wv,
                            const uint16_t* wo, const float* mask, int mask_mode, uint16_t* output, int B, int S, int dModel, int heads);
/* The forms above gather [Wq|Wk|Wv] into the workspace on every call (3 dModel^2 elements read and written).  For constant
 * weights, pack once into a caller-owned [dModel, 3 dModel] buffer (elem_bytes 4 for fp32, 2 for fp16 / bf16) and call the
 * *_packed forms, which read it in place: the concatenated weight of SimdGemm.SgemmConcatenatedProjections
 * (Engines/Simd/SimdGemm.NParallelSmallM.cs:95-109) and of the fused QKV GEMM in CpuEngine.MultiHeadAttention.cs:358-420. */
AIDN_API int aidn_mi355_mha_pack_qkv(void* ctx, void* stream, const void* wq, const void* wk, const void* wv, void* packed,
                            int dModel, int elem_bytes);
AIDN_API int aidn_mi355_mha_fwd_packed_f32(void* ctx, void* stream, const float* input, const float* wqkv, const float* wo,
                                  const float* mask, int mask_mode, float* output, int B, int S, int dModel, int heads);
AIDN_API int aidn_mi355_mha_fwd_packed_f16(void* ctx, void* stream, const uint16_t* input, const uint16_t* wqkv, const uint16_t* wo,
                                  const float* mask, int mask_mode, uint16_t* output, int B, int S, int dModel, int heads);
AIDN_API int aidn_mi355_mha_fwd_packed_bf16(void* ctx, void* stream, const uint16_t* input, const uint16_t* wqkv, const uint16_t* wo,
                                   const float* mask, int mask_mode, uint16_t* output, int B, int S, int dModel, int heads);

/* ---- test / tuning hook --------------------------------------------------------------------------------
 * Forces the GEMM tile edge (64, 128 or 256; 129 / 65 = 128 / 64 on the direct-to-LDS kernel; 192 / 193 / 130 / 131 = the 256 x 192 /
 * 256 x 128 / 128 x 128 (four-stage ring) / 128 x 128 (two-stage ring) tiles of the 16-bit 16x16x32 kernel, whole column tiles only; 0 = automatic choice) for subsequent calls on this context, so the parity suite can exercise every kernel instance.  No counterpart in the
 * reference. */
AIDN_API int aidn_mi355_set_gemm_tile(void* ctx, int tile);
/* enabled == 0 routes every attention shape through the general kernel (the head-dim-128 16-bit fast
 * paths are then not taken), so the parity suite can hold the kernels against each other; unsplit
 * head-dim-128 prefill on dense 16-bit arrays has two kernels (the software-pipelined one is the default, the
 * phase-structured one takes the other layouts): enabled == 2 pins the phase-structured one, enabled == 3 the
 * software-pipelined one wherever it applies (each of the three is checked against the others); at head dimension 256
 * enabled == 2 pins the older 32-key-tile form in place of the 64-key-tile kernel.  Per context.
 * No counterpart in the reference. */
AIDN_API int aidn_mi355_set_attention_fast_path(void* ctx, int enabled);

#ifdef __cplusplus
}
#endif
#endif /* AIDOTNET_MI355_H */
