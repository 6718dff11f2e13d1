// Capability interface for backends with bf16 matrix products and reduced-precision fused attention: the sibling of
// IGpuHalfPrecisionBackend (Engines/Gpu/IGpuHalfPrecisionBackend.cs:21-114), which covers fp16 only.  The reference has no bf16
// member on any backend interface today (its planner widens bf16 tensors to fp32, Engines/Gpu/GpuPrecisionPolicy.cs:497-532);
// consumers downcast (`backend as IGpuBFloat16Backend`) exactly as they do for the fp16 interface.
// NOT COMPILED in this repository (no .NET toolchain in its build image).
using AiDotNet.Tensors.Engines.DirectGpu;

namespace AiDotNet.Tensors.Engines.Gpu
{
    public interface IGpuBFloat16Backend
    {
        /// <summary>True when the backend ships bf16 matrix products (bf16 operands, fp32 accumulation).</summary>
        bool SupportsBf16Gemm { get; }

        /// <summary>C = A · B with A [m,k], B [k,n] and C [m,n] all bf16; fp32 accumulation, one round-to-nearest-even narrow
        /// (the arithmetic of the CPU kernel, Engines/Simd/BFloat16Kernels.cs:144-211, NumericOperations/BFloat16.cs:64-90).</summary>
        void Bf16Gemm(IGpuBuffer aBf16, IGpuBuffer bBf16, IGpuBuffer cBf16, int m, int n, int k);

        /// <summary>Mixed-precision product: A, B bf16, accumulator and C fp32 (the bf16 counterpart of GemmFp16In32fOut).</summary>
        void GemmBf16In32fOut(IGpuBuffer aBf16, IGpuBuffer bBf16, IGpuBuffer cFp32, int m, int n, int k);

        /// <summary>C = A · B in fp16 or bf16 (fp32 accumulation, C in the inputs' type), then RopeInterleaved over the first
        /// <paramref name="ropeCols"/> columns of C (heads of <paramref name="headDim"/> side by side; row r at position
        /// startPosition + r % seqLen): a decode-step projection and its rotation in one call.</summary>
        void GemmRopeReducedPrecision(GpuScalarType inputType, IGpuBuffer a, IGpuBuffer b, IGpuBuffer c, int m, int n, int k,
            IGpuBuffer cos, IGpuBuffer sin, int headDim, int ropeCols, int seqLen, int startPosition);

        /// <summary>fp32 -> bf16 storage conversion, round-to-nearest-even, NaN keeps a quiet bit (BFloat16.FromFloat).</summary>
        void ConvertToBf16(IGpuBuffer inputFp32, IGpuBuffer outputBf16, int size);

        /// <summary>bf16 -> fp32 (exact).</summary>
        void ConvertBf16ToFp32(IGpuBuffer inputBf16, IGpuBuffer outputFp32, int size);

        /// <summary>Fused attention forward on fp16 or bf16 Q, K, V ([batch, heads, seq, headDim], K and V with numKVHeads heads):
        /// fp32 softmax and accumulation; the output is fp32, or the input type when <paramref name="outputIsInputType"/>;
        /// <paramref name="softmaxStats"/> (fp32 log-sum-exp per row) may be null.  Key j is masked for query i iff isCausal and
        /// j &gt; i + causalQueryOffset (0 = top-left rule of FlashAttentionV2, seqK - seqQ = bottom-right rule of
        /// ScaledDotProductAttention).</summary>
        void FlashAttentionReducedPrecision(GpuScalarType inputType, IGpuBuffer query, IGpuBuffer key, IGpuBuffer value, IGpuBuffer output, IGpuBuffer? softmaxStats,
            int batch, int numHeads, int numKVHeads, int seqQ, int seqK, int headDim, float scale, bool isCausal, int causalQueryOffset, bool outputIsInputType);

        /// <summary>One query row per (batch, head) against a dense [batch, numKVHeads, cacheLen, headDim] fp16 or bf16 cache.</summary>
        void DecodeAttentionReducedPrecision(GpuScalarType inputType, IGpuBuffer query, IGpuBuffer keyCache, IGpuBuffer valueCache, IGpuBuffer output,
            int batch, int numHeads, int numKVHeads, int cacheLen, int headDim, float scale, bool outputIsInputType, int splits = 0);
    }
}
