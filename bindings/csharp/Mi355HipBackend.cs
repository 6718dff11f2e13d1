// The backend decorator that puts libaidotnet_mi355.so behind the reference's GPU-backend slot.
//
// HipBackend is sealed (Engines/DirectGpu/HIP/HipBackend.cs:33), so the non-invasive route is the decorator base the reference
// ships (Engines/Gpu/DelegatingGpuBackend.cs:12-26): every member not overridden here keeps going to the wrapped HipBackend.
// Argument checks stay on the managed side, with the reference's exception types and messages (GpuKernelGuards.cs:14-70,
// HipBackend.cs:6126-6148, 6268-6282); the native layer repeats the cheap ones and reports them as status 1001.
// The reference's contract "result ready on return" (HipBackend.cs:1444-1446) is kept: every member synchronises the stream.
// NOT COMPILED in this repository (no .NET toolchain in its build image); tests/test_csharp_binding.py checks that every native
// call made here exists in Mi355Native.cs with that argument count.
using System;
using System.Collections.Generic;
using AiDotNet.Tensors.Engines.Gpu;

namespace AiDotNet.Tensors.Engines.DirectGpu.HIP
{
    internal sealed class Mi355HipBackend : DelegatingGpuBackend, IGpuHalfPrecisionBackend, IGpuBFloat16Backend, IGpuPrecisionBackend, IDisposable
    {
        private readonly HipBackend _hip;
        private readonly IntPtr _ctx;
        private readonly IntPtr _stream;     // the wrapped backend's hipStream_t (HipBackend.DefaultStream, HipBackend.cs:208-222; IGpuStream.Handle)
        private bool _disposed;

        /// <param name="inner">The HIP backend whose stream, allocator and remaining kernels are kept.</param>
        /// <param name="deviceIndex">The factory's device index (HipBackend selects it in its constructor, HipBackend.cs:246).</param>
        public Mi355HipBackend(HipBackend inner, int deviceIndex) : base(inner)
        {
            _hip = inner;
            Mi355Native.Check(IntPtr.Zero, Mi355Native.aidn_mi355_create(deviceIndex, out _ctx), "aidn_mi355_create");
            _stream = inner.DefaultStream.Handle;
        }

        public override string BackendName => Inner.BackendName + "+mi355";

        private void Sync(string op) => Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_sync(_ctx, _stream), op);

        private static void Positive(int m, int n, int k, string op)
        {
            if (m <= 0 || n <= 0 || k <= 0)
                throw new ArgumentOutOfRangeException(nameof(m), $"{op}: M, N, K must all be > 0 (got M={m}, N={n}, K={k}).");
        }

        // ------------------------------------------------------------------ fp32 GEMM (IDirectGpuBackend.cs:160-222)
        public override void Gemm(IGpuBuffer A, IGpuBuffer B, IGpuBuffer C, int M, int N, int K, float alpha = 1.0f, float beta = 0.0f)
        {
            Positive(M, N, K, nameof(Gemm));
            GpuKernelGuards.Capacity(A, (long)M * K, nameof(A), nameof(Gemm));
            GpuKernelGuards.Capacity(B, (long)K * N, nameof(B), nameof(Gemm));
            GpuKernelGuards.Capacity(C, (long)M * N, nameof(C), nameof(Gemm));
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_sgemm(_ctx, _stream, A.Handle, B.Handle, C.Handle, M, N, K, alpha, beta, 0), nameof(Gemm));
            Sync(nameof(Gemm));
        }

        public override IGpuBuffer MatMul(IGpuBuffer A, IGpuBuffer B, int M, int N, int K)
        {
            var c = AllocateBuffer(M * N);
            try { Gemm(A, B, c, M, N, K, 1.0f, 0.0f); }
            catch { c.Dispose(); throw; }
            return c;
        }

        public override void MatMulTransposed(IGpuBuffer A, IGpuBuffer B, IGpuBuffer C, int M, int N, int K, float alpha = 1.0f, float beta = 0.0f)
        {
            Positive(M, N, K, nameof(MatMulTransposed));
            GpuKernelGuards.Capacity(A, (long)M * K, nameof(A), nameof(MatMulTransposed));
            GpuKernelGuards.Capacity(B, (long)N * K, nameof(B), nameof(MatMulTransposed));      // B is stored [N, K]
            GpuKernelGuards.Capacity(C, (long)M * N, nameof(C), nameof(MatMulTransposed));
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_sgemm(_ctx, _stream, A.Handle, B.Handle, C.Handle, M, N, K, alpha, beta, 1), nameof(MatMulTransposed));
            Sync(nameof(MatMulTransposed));
        }

        public override void BatchedGemm(IGpuBuffer A, IGpuBuffer B, IGpuBuffer C, int M, int N, int K, int batchCount, float alpha = 1.0f, float beta = 0.0f)
        {
            Positive(M, N, K, nameof(BatchedGemm));
            if (batchCount <= 0) throw new ArgumentOutOfRangeException(nameof(batchCount), $"{nameof(BatchedGemm)}: batchCount must be > 0 (got {batchCount}).");
            GpuKernelGuards.Capacity(A, (long)batchCount * M * K, nameof(A), nameof(BatchedGemm));
            GpuKernelGuards.Capacity(B, (long)batchCount * K * N, nameof(B), nameof(BatchedGemm));
            GpuKernelGuards.Capacity(C, (long)batchCount * M * N, nameof(C), nameof(BatchedGemm));
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_sgemm_batched(_ctx, _stream, A.Handle, B.Handle, C.Handle, M, N, K, batchCount, alpha, beta), nameof(BatchedGemm));
            Sync(nameof(BatchedGemm));
        }

        // ------------------------------------------------------------------ fused projection epilogues (IDirectGpuBackend.cs:227-275)
        // One kernel where HipBackend runs a GEMM, a bias kernel and an activation kernel (HipBackend.cs:1637-1785).
        private IGpuBuffer GemmBiasAct(IGpuBuffer A, IGpuBuffer B, IGpuBuffer bias, int M, int N, int K, FusedActivationType act, float param, string op)
        {
            Positive(M, N, K, op);
            GpuKernelGuards.Capacity(A, (long)M * K, nameof(A), op);
            GpuKernelGuards.Capacity(B, (long)K * N, nameof(B), op);
            GpuKernelGuards.Capacity(bias, N, nameof(bias), op);
            var c = AllocateBuffer(M * N);
            try
            {
                Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_sgemm_bias_act(_ctx, _stream, A.Handle, B.Handle, bias.Handle, c.Handle, M, N, K, (int)act, param), op);
                Sync(op);
            }
            catch { c.Dispose(); throw; }
            return c;
        }

        public override IGpuBuffer GemmBias(IGpuBuffer A, IGpuBuffer B, IGpuBuffer bias, int M, int N, int K)
            => GemmBiasAct(A, B, bias, M, N, K, FusedActivationType.None, 0.0f, nameof(GemmBias));
        public override IGpuBuffer GemmBiasRelu(IGpuBuffer A, IGpuBuffer B, IGpuBuffer bias, int M, int N, int K)
            => GemmBiasAct(A, B, bias, M, N, K, FusedActivationType.ReLU, 0.0f, nameof(GemmBiasRelu));
        public override IGpuBuffer GemmBiasGelu(IGpuBuffer A, IGpuBuffer B, IGpuBuffer bias, int M, int N, int K)
            => GemmBiasAct(A, B, bias, M, N, K, FusedActivationType.GELU, 0.0f, nameof(GemmBiasGelu));
        public override IGpuBuffer GemmBiasSigmoid(IGpuBuffer A, IGpuBuffer B, IGpuBuffer bias, int M, int N, int K)
            => GemmBiasAct(A, B, bias, M, N, K, FusedActivationType.Sigmoid, 0.0f, nameof(GemmBiasSigmoid));
        public override IGpuBuffer GemmBiasTanh(IGpuBuffer A, IGpuBuffer B, IGpuBuffer bias, int M, int N, int K)
            => GemmBiasAct(A, B, bias, M, N, K, FusedActivationType.Tanh, 0.0f, nameof(GemmBiasTanh));
        public override IGpuBuffer GemmBiasSwish(IGpuBuffer A, IGpuBuffer B, IGpuBuffer bias, int M, int N, int K)
            => GemmBiasAct(A, B, bias, M, N, K, FusedActivationType.Swish, 0.0f, nameof(GemmBiasSwish));
        public override IGpuBuffer GemmBiasLeakyRelu(IGpuBuffer A, IGpuBuffer B, IGpuBuffer bias, int M, int N, int K, float alpha = 0.01f)
            => GemmBiasAct(A, B, bias, M, N, K, FusedActivationType.LeakyReLU, alpha, nameof(GemmBiasLeakyRelu));

        // ------------------------------------------------------------------ fp16 (IGpuHalfPrecisionBackend.cs:21-114)
        public bool SupportsHgemm => true;

        public void Hgemm(IGpuBuffer aFp16, IGpuBuffer bFp16, IGpuBuffer cFp16, int m, int n, int k)
        {
            Positive(m, n, k, nameof(Hgemm));
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_hgemm_f16out(_ctx, _stream, aFp16.Handle, bFp16.Handle, cFp16.Handle, m, n, k), nameof(Hgemm));
            Sync(nameof(Hgemm));
        }

        public void GemmFp16In32fOut(IGpuBuffer aFp16, IGpuBuffer bFp16, IGpuBuffer cFp32, int m, int n, int k)
        {
            Positive(m, n, k, nameof(GemmFp16In32fOut));
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_hgemm_f32out(_ctx, _stream, aFp16.Handle, bFp16.Handle, cFp32.Handle, m, n, k), nameof(GemmFp16In32fOut));
            Sync(nameof(GemmFp16In32fOut));
        }

        // the members of the interface that are not on this path stay with the wrapped backend
        public bool SupportsFp16FusedBackward => _hip.SupportsFp16FusedBackward;
        public void MatMulBackwardFp16Fused(IGpuBuffer gradCFp16, IGpuBuffer aFp16, IGpuBuffer bFp16, IGpuBuffer gradAOut, IGpuBuffer gradBOut,
            int m, int n, int k, bool gradOutHalf) => _hip.MatMulBackwardFp16Fused(gradCFp16, aFp16, bFp16, gradAOut, gradBOut, m, n, k, gradOutHalf);
        public bool SupportsFp16NativeOps => _hip.SupportsFp16NativeOps;
        public void Fp16Softmax(IGpuBuffer input, IGpuBuffer output, int rows, int cols) => _hip.Fp16Softmax(input, output, rows, cols);
        public void Fp16LayerNorm(IGpuBuffer input, IGpuBuffer gamma, IGpuBuffer beta, IGpuBuffer output, IGpuBuffer meanFp32, IGpuBuffer varFp32,
            int rows, int cols, float eps) => _hip.Fp16LayerNorm(input, gamma, beta, output, meanFp32, varFp32, rows, cols, eps);
        public bool Fp16Im2colAvailable => _hip.Fp16Im2colAvailable;
        public void Im2colKNFp16(IGpuBuffer input, IGpuBuffer outputHalf, int batch, int channels, int height, int width,
            int kernelH, int kernelW, int strideH, int strideW, int padH, int padW, int dilationH, int dilationW)
            => _hip.Im2colKNFp16(input, outputHalf, batch, channels, height, width, kernelH, kernelW, strideH, strideW, padH, padW, dilationH, dilationW);

        // ------------------------------------------------------------------ bf16 (IGpuBFloat16Backend.cs)
        public bool SupportsBf16Gemm => true;

        public void Bf16Gemm(IGpuBuffer aBf16, IGpuBuffer bBf16, IGpuBuffer cBf16, int m, int n, int k)
        {
            Positive(m, n, k, nameof(Bf16Gemm));
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_bf16gemm_bf16out(_ctx, _stream, aBf16.Handle, bBf16.Handle, cBf16.Handle, m, n, k), nameof(Bf16Gemm));
            Sync(nameof(Bf16Gemm));
        }

        public void GemmBf16In32fOut(IGpuBuffer aBf16, IGpuBuffer bBf16, IGpuBuffer cFp32, int m, int n, int k)
        {
            Positive(m, n, k, nameof(GemmBf16In32fOut));
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_bf16gemm_f32out(_ctx, _stream, aBf16.Handle, bBf16.Handle, cFp32.Handle, m, n, k), nameof(GemmBf16In32fOut));
            Sync(nameof(GemmBf16In32fOut));
        }

        public void GemmRopeReducedPrecision(GpuScalarType inputType, IGpuBuffer a, IGpuBuffer b, IGpuBuffer c, int m, int n, int k,
            IGpuBuffer cos, IGpuBuffer sin, int headDim, int ropeCols, int seqLen, int startPosition)
        {
            Positive(m, n, k, nameof(GemmRopeReducedPrecision));
            if (headDim <= 0 || seqLen <= 0) throw new ArgumentOutOfRangeException(nameof(headDim), "RoPE dimensions must be positive.");
            if ((headDim & 1) != 0) throw new ArgumentException("headDim must be even.", nameof(headDim));
            if (startPosition < 0) throw new ArgumentOutOfRangeException(nameof(startPosition));
            if (ropeCols < 0 || ropeCols > n || ropeCols % headDim != 0 || (n & 1) != 0)
                throw new ArgumentException("ropeCols must be a multiple of headDim within n, and n even.", nameof(ropeCols));
            int status = inputType switch
            {
                GpuScalarType.Float16 => Mi355Native.aidn_mi355_hgemm_rope(_ctx, _stream, a.Handle, b.Handle, c.Handle, m, n, k, cos.Handle, sin.Handle, headDim, ropeCols, seqLen, startPosition),
                GpuScalarType.BFloat16 => Mi355Native.aidn_mi355_bf16gemm_rope(_ctx, _stream, a.Handle, b.Handle, c.Handle, m, n, k, cos.Handle, sin.Handle, headDim, ropeCols, seqLen, startPosition),
                _ => throw new NotSupportedException($"{nameof(GemmRopeReducedPrecision)}: input type must be Float16 or BFloat16 (got {inputType})."),
            };
            Mi355Native.Check(_ctx, status, nameof(GemmRopeReducedPrecision));
            Sync(nameof(GemmRopeReducedPrecision));
        }

        public void ConvertToBf16(IGpuBuffer inputFp32, IGpuBuffer outputBf16, int size)
        {
            if (size <= 0) throw new ArgumentOutOfRangeException(nameof(size));
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_convert_f32_to_bf16(_ctx, _stream, inputFp32.Handle, outputBf16.Handle, size), nameof(ConvertToBf16));
            Sync(nameof(ConvertToBf16));
        }

        public void ConvertBf16ToFp32(IGpuBuffer inputBf16, IGpuBuffer outputFp32, int size)
        {
            if (size <= 0) throw new ArgumentOutOfRangeException(nameof(size));
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_convert_bf16_to_f32(_ctx, _stream, inputBf16.Handle, outputFp32.Handle, size), nameof(ConvertBf16ToFp32));
            Sync(nameof(ConvertBf16ToFp32));
        }

        public void FlashAttentionReducedPrecision(GpuScalarType inputType, IGpuBuffer query, IGpuBuffer key, IGpuBuffer value, IGpuBuffer output, IGpuBuffer? softmaxStats,
            int batch, int numHeads, int numKVHeads, int seqQ, int seqK, int headDim, float scale, bool isCausal, int causalQueryOffset, bool outputIsInputType)
        {
            AttentionDims(batch, numHeads, seqQ, seqK, headDim, nameof(FlashAttentionReducedPrecision));
            int kvHeads = numKVHeads > 0 ? numKVHeads : numHeads;
            GpuKernelGuards.Gqa(numHeads, kvHeads, nameof(FlashAttentionReducedPrecision));
            var d = new AidnAttnDesc { B = batch, H = numHeads, Hkv = kvHeads, Sq = seqQ, Sk = seqK, D = headDim, Scale = scale,
                                       Causal = isCausal ? 1 : 0, CausalQueryOffset = causalQueryOffset, OutIs16Bit = outputIsInputType ? 1 : 0 };
            IntPtr lse = softmaxStats?.Handle ?? IntPtr.Zero;
            int status = inputType switch
            {
                GpuScalarType.Float16 => Mi355Native.aidn_mi355_attn_fwd_f16(_ctx, _stream, ref d, query.Handle, key.Handle, value.Handle, output.Handle, lse, IntPtr.Zero, IntPtr.Zero, IntPtr.Zero),
                GpuScalarType.BFloat16 => Mi355Native.aidn_mi355_attn_fwd_bf16(_ctx, _stream, ref d, query.Handle, key.Handle, value.Handle, output.Handle, lse, IntPtr.Zero, IntPtr.Zero, IntPtr.Zero),
                _ => throw new NotSupportedException($"{nameof(FlashAttentionReducedPrecision)}: input type must be Float16 or BFloat16 (got {inputType})."),
            };
            Mi355Native.Check(_ctx, status, nameof(FlashAttentionReducedPrecision));
            Sync(nameof(FlashAttentionReducedPrecision));
        }

        public void DecodeAttentionReducedPrecision(GpuScalarType inputType, IGpuBuffer query, IGpuBuffer keyCache, IGpuBuffer valueCache, IGpuBuffer output,
            int batch, int numHeads, int numKVHeads, int cacheLen, int headDim, float scale, bool outputIsInputType, int splits = 0)
        {
            AttentionDims(batch, numHeads, 1, cacheLen, headDim, nameof(DecodeAttentionReducedPrecision));
            int kvHeads = numKVHeads > 0 ? numKVHeads : numHeads;
            GpuKernelGuards.Gqa(numHeads, kvHeads, nameof(DecodeAttentionReducedPrecision));
            var d = new AidnAttnDesc { B = batch, H = numHeads, Hkv = kvHeads, Sq = 1, Sk = cacheLen, D = headDim, Scale = scale, OutIs16Bit = outputIsInputType ? 1 : 0 };
            int status = inputType switch
            {
                GpuScalarType.Float16 => Mi355Native.aidn_mi355_attn_decode_f16(_ctx, _stream, ref d, query.Handle, keyCache.Handle, valueCache.Handle, output.Handle, IntPtr.Zero, splits),
                GpuScalarType.BFloat16 => Mi355Native.aidn_mi355_attn_decode_bf16(_ctx, _stream, ref d, query.Handle, keyCache.Handle, valueCache.Handle, output.Handle, IntPtr.Zero, splits),
                _ => throw new NotSupportedException($"{nameof(DecodeAttentionReducedPrecision)}: input type must be Float16 or BFloat16 (got {inputType})."),
            };
            Mi355Native.Check(_ctx, status, nameof(DecodeAttentionReducedPrecision));
            Sync(nameof(DecodeAttentionReducedPrecision));
        }

        // ------------------------------------------------------------------ precision capabilities (DirectGpuPrecisionCapabilities.cs:60-101)
        public IReadOnlyList<GpuPrecisionCapability> GetPrecisionCapabilities(GpuPrecisionOperation operation)
        {
            // what the HIP backend reports, with the matrix products marked Native (hand-written kernels, no vendor library) and a
            // bf16 row for MatMul (storage and multiply bf16, accumulate and output fp32, operand bytes halved)
            bool gemm = operation is GpuPrecisionOperation.MatMul or GpuPrecisionOperation.MatMulTransposed or GpuPrecisionOperation.BatchMatMul;
            if (!gemm) return _hip.GetPrecisionCapabilities(operation);
            return GpuPrecisionCapabilityCatalog.Create(
                supportsFp16: operation == GpuPrecisionOperation.MatMul,
                fp16Implementation: GpuPrecisionImplementation.Native,
                fp16ReducesStorageBytes: true,
                fp32Implementation: GpuPrecisionImplementation.Native,
                supportsBFloat16: operation == GpuPrecisionOperation.MatMul);      // new optional argument, see reference_changes.patch
        }

        // ------------------------------------------------------------------ storage conversions (IDirectGpuBackend.cs:1876-1911)
        public override void ConvertToFp16(IGpuBuffer input, IGpuBuffer output, int size)
        {
            if (size <= 0) throw new ArgumentOutOfRangeException(nameof(size));
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_convert_f32_to_f16(_ctx, _stream, input.Handle, output.Handle, size), nameof(ConvertToFp16));
            Sync(nameof(ConvertToFp16));
        }

        public override void ConvertToFp32(IGpuBuffer input, IGpuBuffer output, int size)
        {
            if (size <= 0) throw new ArgumentOutOfRangeException(nameof(size));
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_convert_f16_to_f32(_ctx, _stream, input.Handle, output.Handle, size), nameof(ConvertToFp32));
            Sync(nameof(ConvertToFp32));
        }

        // ------------------------------------------------------------------ attention (IDirectGpuBackend.cs:1395-1471)
        private static void AttentionDims(int batch, int numHeads, int seqQ, int seqK, int headDim, string op)
        {
            if (batch <= 0 || numHeads <= 0 || seqQ <= 0 || seqK <= 0 || headDim <= 0)
                throw new ArgumentOutOfRangeException(nameof(batch), "Attention dimensions must be positive.");
            if (headDim > GpuKernelGuards.MaxHeadDim)
                throw new ArgumentOutOfRangeException(nameof(headDim), $"{op}: headDim must be in [1, {GpuKernelGuards.MaxHeadDim}] (got {headDim}).");
        }

        public override void ScaledDotProductAttention(IGpuBuffer query, IGpuBuffer key, IGpuBuffer value,
            IGpuBuffer output, IGpuBuffer? attentionWeights, IGpuBuffer? mask,
            int batch, int numHeads, int seqQ, int seqK, int headDim, float scale, bool isCausal, float softcap = 0.0f, int numKVHeads = 0)
        {
            AttentionDims(batch, numHeads, seqQ, seqK, headDim, nameof(ScaledDotProductAttention));
            int kvHeads = numKVHeads > 0 ? numKVHeads : numHeads;
            if (numHeads % kvHeads != 0) throw new ArgumentException("numHeads must be an integer multiple of numKVHeads.", nameof(numKVHeads));
            long qElems = (long)batch * numHeads * seqQ * headDim, kvElems = (long)batch * kvHeads * seqK * headDim, wElems = (long)batch * numHeads * seqQ * seqK;
            if (query.Size < qElems || key.Size < kvElems || value.Size < kvElems || output.Size < qElems)
                throw new ArgumentException("Attention tensor buffers are smaller than the requested dimensions.");
            if (attentionWeights != null && attentionWeights.Size < wElems) throw new ArgumentException("The attention-weights buffer is too small.", nameof(attentionWeights));
            if (mask != null && mask.Size < (long)seqQ * seqK) throw new ArgumentException("The attention mask must contain at least seqQ * seqK elements.", nameof(mask));
            var d = new AidnAttnDesc
            {
                B = batch, H = numHeads, Hkv = kvHeads, Sq = seqQ, Sk = seqK, D = headDim, Scale = scale,
                Causal = isCausal ? 1 : 0,
                CausalQueryOffset = seqK - seqQ,                                    // bottom-right alignment (HipAttentionKernels.cs:69-71)
                Softcap = softcap,
                MaskMode = mask == null ? 0 : (mask.Size >= wElems ? 2 : 1),        // one shared [seqQ, seqK] plane, or the full tensor (HipBackend.cs:6150-6151)
            };
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_attn_fwd_f32(_ctx, _stream, ref d, query.Handle, key.Handle, value.Handle, output.Handle,
                IntPtr.Zero, IntPtr.Zero, mask?.Handle ?? IntPtr.Zero, attentionWeights?.Handle ?? IntPtr.Zero), nameof(ScaledDotProductAttention));
            Sync(nameof(ScaledDotProductAttention));
        }

        public override void FlashAttentionV2(IGpuBuffer query, IGpuBuffer key, IGpuBuffer value,
            IGpuBuffer output, IGpuBuffer softmaxStats,
            int batch, int numHeads, int seqQ, int seqK, int headDim, float scale, bool isCausal,
            IGpuBuffer? attentionBias = null, int biasBatchStride = 0)
        {
            AttentionDims(batch, numHeads, seqQ, seqK, headDim, nameof(FlashAttentionV2));
            long qElems = (long)batch * numHeads * seqQ * headDim, kvElems = (long)batch * numHeads * seqK * headDim;
            if (query.Size < qElems || key.Size < kvElems || value.Size < kvElems || output.Size < qElems)
                throw new ArgumentException("Attention tensor buffers are smaller than the requested dimensions.");
            if (softmaxStats.Size < (long)batch * numHeads * seqQ) throw new ArgumentException("The softmax-statistics buffer is too small.", nameof(softmaxStats));
            var d = new AidnAttnDesc { B = batch, H = numHeads, Hkv = numHeads, Sq = seqQ, Sk = seqK, D = headDim, Scale = scale,
                                       Causal = isCausal ? 1 : 0, CausalQueryOffset = 0,        // top-left rule: key j masked iff j > i (HipAttentionKernels.cs:199)
                                       BiasBatchStride = biasBatchStride };
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_attn_fwd_f32(_ctx, _stream, ref d, query.Handle, key.Handle, value.Handle, output.Handle,
                softmaxStats.Handle, attentionBias?.Handle ?? IntPtr.Zero, IntPtr.Zero, IntPtr.Zero), nameof(FlashAttentionV2));
            Sync(nameof(FlashAttentionV2));
        }

        public override void FlashAttention(IGpuBuffer query, IGpuBuffer key, IGpuBuffer value,
            IGpuBuffer output, IGpuBuffer? mask, int batch, int numHeads, int seqLen, int headDim, float scale, bool isCausal)
        {
            // as the reference: the V2 kernel with a scratch statistics buffer; `mask` is not read (HipBackend.cs:6250-6259)
            using var stats = AllocateBuffer(batch * numHeads * seqLen);
            FlashAttentionV2(query, key, value, output, stats, batch, numHeads, seqLen, seqLen, headDim, scale, isCausal);
        }

        /// <summary>Single-sequence decode over K/V laid out [seqLen, kvHeads, headDim] (HipBackend.cs:919-965).</summary>
        public IGpuBuffer FlashDecode(IGpuBuffer q, IGpuBuffer k, IGpuBuffer v, int heads, int kvHeads, int headDim, int seqLen, float scale, int splits = 0)
        {
            GpuKernelGuards.FlashDecode(heads, kvHeads, headDim, seqLen, nameof(FlashDecode));
            GpuKernelGuards.Capacity(q, (long)heads * headDim, nameof(q), nameof(FlashDecode));
            GpuKernelGuards.Capacity(k, (long)seqLen * kvHeads * headDim, nameof(k), nameof(FlashDecode));
            GpuKernelGuards.Capacity(v, (long)seqLen * kvHeads * headDim, nameof(v), nameof(FlashDecode));
            var o = AllocateBuffer(heads * headDim);
            try
            {
                var d = new AidnAttnDesc { B = 1, H = heads, Hkv = kvHeads, Sq = 1, Sk = seqLen, D = headDim, Scale = scale };
                // [seqLen, kvHeads, d]: batch stride unused (B = 1), head stride d, row stride kvHeads * d
                d.QStride0 = (long)heads * headDim; d.QStride1 = headDim; d.QStride2 = headDim;
                d.KStride0 = (long)seqLen * kvHeads * headDim; d.KStride1 = headDim; d.KStride2 = (long)kvHeads * headDim;
                d.VStride0 = d.KStride0; d.VStride1 = d.KStride1; d.VStride2 = d.KStride2;
                d.OStride0 = (long)heads * headDim; d.OStride1 = headDim; d.OStride2 = headDim;
                Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_attn_decode_f32(_ctx, _stream, ref d, q.Handle, k.Handle, v.Handle, o.Handle, IntPtr.Zero, splits), nameof(FlashDecode));
                Sync(nameof(FlashDecode));
            }
            catch { o.Dispose(); throw; }
            return o;
        }

        public override void RopeInterleaved(IGpuBuffer input, IGpuBuffer cos, IGpuBuffer sin, IGpuBuffer output, int rows, int headDim, int seqLen, int startPosition)
        {
            if (rows <= 0 || headDim <= 0 || seqLen <= 0) throw new ArgumentOutOfRangeException(nameof(rows), "RoPE dimensions must be positive.");
            if ((headDim & 1) != 0) throw new ArgumentException("headDim must be even.", nameof(headDim));
            if (startPosition < 0) throw new ArgumentOutOfRangeException(nameof(startPosition));
            GpuKernelGuards.Capacity(input, (long)rows * headDim, nameof(input), nameof(RopeInterleaved));
            GpuKernelGuards.Capacity(output, (long)rows * headDim, nameof(output), nameof(RopeInterleaved));
            GpuKernelGuards.Capacity(cos, (long)(startPosition + seqLen) * (headDim / 2), nameof(cos), nameof(RopeInterleaved));
            GpuKernelGuards.Capacity(sin, (long)(startPosition + seqLen) * (headDim / 2), nameof(sin), nameof(RopeInterleaved));
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_rope_interleaved_f32(_ctx, _stream, input.Handle, cos.Handle, sin.Handle, output.Handle, rows, headDim, seqLen, startPosition), nameof(RopeInterleaved));
            Sync(nameof(RopeInterleaved));
        }

        // ------------------------------------------------------------------ paged attention (IDirectGpuBackend.cs:3614-3633)
        private IGpuBuffer Paged(IGpuBuffer q, IGpuBuffer kcache, IGpuBuffer vcache, IGpuBuffer blockTable, int heads, int kvHeads, int headDim, int blockSize,
            int numQueries, int keyLen, int startPos, float scale, bool decode, string op)
        {
            GpuKernelGuards.Attention(heads, headDim, blockSize, decode ? keyLen : numQueries, op);
            GpuKernelGuards.Gqa(heads, kvHeads, op);
            if (!decode && startPos < 0) throw new ArgumentOutOfRangeException(nameof(startPos), $"{op}: startPos must be >= 0 (got {startPos}).");
            GpuKernelGuards.Capacity(q, (long)numQueries * heads * headDim, nameof(q), op);
            GpuKernelGuards.Capacity(blockTable, (keyLen + blockSize - 1) / blockSize, nameof(blockTable), op);
            var o = AllocateBuffer(numQueries * heads * headDim);
            try
            {
                int status = decode
                    ? Mi355Native.aidn_mi355_paged_attn_decode_f32(_ctx, _stream, q.Handle, kcache.Handle, vcache.Handle, blockTable.Handle, o.Handle, heads, kvHeads, headDim, blockSize, keyLen, scale, 0)
                    : Mi355Native.aidn_mi355_paged_attn_prefill_f32(_ctx, _stream, q.Handle, kcache.Handle, vcache.Handle, blockTable.Handle, o.Handle, heads, kvHeads, headDim, blockSize, numQueries, startPos, scale);
                Mi355Native.Check(_ctx, status, op);
                Sync(op);
            }
            catch { o.Dispose(); throw; }
            return o;
        }

        public override IGpuBuffer PagedAttentionDecode(IGpuBuffer q, IGpuBuffer kcache, IGpuBuffer vcache, IGpuBuffer blockTable, int heads, int headDim, int blockSize, int seqLen, float scale)
            => Paged(q, kcache, vcache, blockTable, heads, heads, headDim, blockSize, 1, seqLen, 0, scale, true, nameof(PagedAttentionDecode));
        public override IGpuBuffer PagedAttentionDecodeGqa(IGpuBuffer q, IGpuBuffer kcache, IGpuBuffer vcache, IGpuBuffer blockTable, int heads, int kvHeads, int headDim, int blockSize, int seqLen, float scale)
            => Paged(q, kcache, vcache, blockTable, heads, kvHeads, headDim, blockSize, 1, seqLen, 0, scale, true, nameof(PagedAttentionDecodeGqa));
        public override IGpuBuffer PagedAttentionPrefill(IGpuBuffer q, IGpuBuffer kcache, IGpuBuffer vcache, IGpuBuffer blockTable, int heads, int headDim, int blockSize, int numQueries, int startPos, float scale)
            => Paged(q, kcache, vcache, blockTable, heads, heads, headDim, blockSize, numQueries, startPos + numQueries, startPos, scale, false, nameof(PagedAttentionPrefill));
        public override IGpuBuffer PagedAttentionPrefillGqa(IGpuBuffer q, IGpuBuffer kcache, IGpuBuffer vcache, IGpuBuffer blockTable, int heads, int kvHeads, int headDim, int blockSize, int numQueries, int startPos, float scale)
            => Paged(q, kcache, vcache, blockTable, heads, kvHeads, headDim, blockSize, numQueries, startPos + numQueries, startPos, scale, false, nameof(PagedAttentionPrefillGqa));

        // ------------------------------------------------------------------ engine-level helpers (called by DirectGpuTensorEngine, no interface member today)
        /// <summary>C = act(A * widen(B_f16) + bias): the GPU form of SimdGemm.SgemmFp16WeightB (SimdGemm.Fp16Weight.cs:22-91).</summary>
        public void GemmFp16Weight(IGpuBuffer aFp32, IGpuBuffer bFp16, IGpuBuffer? bias, IGpuBuffer cFp32, int m, int n, int k, FusedActivationType activation = FusedActivationType.None, float activationParam = 0.0f)
        {
            Positive(m, n, k, nameof(GemmFp16Weight));
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_sgemm_f16weight(_ctx, _stream, aFp32.Handle, bFp16.Handle, bias?.Handle ?? IntPtr.Zero, cFp32.Handle, m, n, k, (int)activation, activationParam), nameof(GemmFp16Weight));
            Sync(nameof(GemmFp16Weight));
        }

        /// <summary>Bytes of the packed form of a [K, N] weight (kind 0 fp32, 1 fp16, 2 bf16): what the engine's PrePackedB cache entry allocates.</summary>
        public long PackedWeightBytes(int kind, int k, int n, bool transB = false) => checked((long)Mi355Native.aidn_mi355_packed_b_bytes(kind, k, n, transB ? 1 : 0));

        public void PackWeight(int kind, IGpuBuffer b, int k, int n, bool transB, IGpuBuffer packed)
        {
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_pack_b(_ctx, _stream, kind, b.Handle, k, n, transB ? 1 : 0, packed.Handle), nameof(PackWeight));
            Sync(nameof(PackWeight));
        }

        public void GemmPackedWeight(int kind, IGpuBuffer a, IGpuBuffer packedB, IGpuBuffer? bias, IGpuBuffer c, bool outputIsFp32, int m, int n, int k, bool transB = false,
            FusedActivationType activation = FusedActivationType.None, float activationParam = 0.0f)
        {
            Positive(m, n, k, nameof(GemmPackedWeight));
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_gemm_packed_b(_ctx, _stream, kind, a.Handle, packedB.Handle, bias?.Handle ?? IntPtr.Zero, c.Handle,
                outputIsFp32 ? 1 : 0, m, n, k, transB ? 1 : 0, (int)activation, activationParam), nameof(GemmPackedWeight));
            Sync(nameof(GemmPackedWeight));
        }

        /// <summary>IEngine.MultiHeadAttentionForward on device buffers (CpuEngine.MultiHeadAttention.cs:68-143); mask fp32, non-zero = keep.</summary>
        public void MultiHeadAttentionForward(IGpuBuffer input, IGpuBuffer wq, IGpuBuffer wk, IGpuBuffer wv, IGpuBuffer wo, IGpuBuffer? mask, bool maskIsFull,
            IGpuBuffer output, int batch, int seq, int dModel, int heads)
        {
            if (batch <= 0 || seq <= 0 || dModel <= 0 || heads <= 0 || dModel % heads != 0)
                throw new ArgumentException($"{nameof(MultiHeadAttentionForward)}: dModel ({dModel}) must be a positive multiple of heads ({heads}).");
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_mha_fwd_f32(_ctx, _stream, input.Handle, wq.Handle, wk.Handle, wv.Handle, wo.Handle,
                mask?.Handle ?? IntPtr.Zero, mask == null ? 0 : (maskIsFull ? 2 : 1), output.Handle, batch, seq, dModel, heads), nameof(MultiHeadAttentionForward));
            Sync(nameof(MultiHeadAttentionForward));
        }

        /// <summary>Grows the library workspace of the backend's stream now, so that calls captured into a HIP graph allocate nothing.</summary>
        public void ReserveWorkspace(long bytes)
        {
            if (bytes < 0) throw new ArgumentOutOfRangeException(nameof(bytes));
            Mi355Native.Check(_ctx, Mi355Native.aidn_mi355_reserve_workspace(_ctx, _stream, (ulong)bytes), nameof(ReserveWorkspace));
        }

        public long WorkspaceBytes => checked((long)Mi355Native.aidn_mi355_workspace_bytes(_ctx, _stream));

        public override void Synchronize() => Sync(nameof(Synchronize));

        public new void Dispose()
        {
            if (_disposed) return;
            _disposed = true;
            Mi355Native.aidn_mi355_destroy(_ctx);
            base.Dispose();
        }
    }
}
