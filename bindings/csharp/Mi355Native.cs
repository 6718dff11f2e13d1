// P/Invoke bindings of libaidotnet_mi355.so (include/aidotnet_mi355.h), one declaration per export.
//
// Written in the style of the reference's own native bindings (Engines/DirectGpu/HIP/HipBlasNative.cs:82-170,
// HipNativeBindings.cs:13-87): cdecl, blittable arguments only, device pointers as IntPtr (IGpuBuffer.Handle,
// Engines/DirectGpu/IDirectGpuBackend.cs:3776-3803), a probe that answers "is the library there" without throwing.
// NOT COMPILED in this repository (there is no .NET toolchain in its build image); tests/test_csharp_binding.py holds every
// declaration below against the header: export present, argument count, blittable type of every argument and of the result.
using System;
using System.Runtime.InteropServices;

namespace AiDotNet.Tensors.Engines.DirectGpu.HIP
{
    /// <summary>aidn_attn_desc of aidotnet_mi355.h: 12 four-byte fields, then 13 eight-byte fields (no padding).</summary>
    [StructLayout(LayoutKind.Sequential)]
    internal struct AidnAttnDesc
    {
        public int B, H, Hkv, Sq, Sk, D;
        public float Scale;
        public int Causal;
        public int CausalQueryOffset;
        public float Softcap;
        public int MaskMode;
        public int OutIs16Bit;
        public long BiasBatchStride;
        // batch, head, row strides in elements; all zero = dense
        public long QStride0, QStride1, QStride2;
        public long KStride0, KStride1, KStride2;
        public long VStride0, VStride1, VStride2;
        public long OStride0, OStride1, OStride2;
    }

    internal static class Mi355Native
    {
        private const string Lib = "aidotnet_mi355";
        private const CallingConvention CC = CallingConvention.Cdecl;

        // status codes of the library (values 1000+); any other non-zero value is a hipError_t
        internal const int Ok = 0, ErrInvalidArgument = 1001, ErrUnsupported = 1002, ErrNoDevice = 1003, ErrOutOfMemory = 1004, ErrWorkspace = 1005;

        // ---- lifetime
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_create(int device, out IntPtr ctx);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_destroy(IntPtr ctx);
        [DllImport(Lib, CallingConvention = CC)] internal static extern IntPtr aidn_mi355_last_error(IntPtr ctx);
        [DllImport(Lib, CallingConvention = CC)] internal static extern IntPtr aidn_mi355_version();
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_sync(IntPtr ctx, IntPtr stream);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_reserve_workspace(IntPtr ctx, IntPtr stream, ulong bytes);
        [DllImport(Lib, CallingConvention = CC)] internal static extern ulong aidn_mi355_workspace_bytes(IntPtr ctx, IntPtr stream);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_release_stream_workspace(IntPtr ctx, IntPtr stream);

        // ---- fp32 GEMM
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_sgemm(IntPtr ctx, IntPtr stream, IntPtr a, IntPtr b, IntPtr c,
            int m, int n, int k, float alpha, float beta, int transB);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_sgemm_batched(IntPtr ctx, IntPtr stream, IntPtr a, IntPtr b, IntPtr c,
            int m, int n, int k, int batch, float alpha, float beta);

        // ---- fused projection epilogues
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_sgemm_bias_act(IntPtr ctx, IntPtr stream, IntPtr a, IntPtr b, IntPtr bias, IntPtr c,
            int m, int n, int k, int activation, float actParam);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_hgemm_bias_act(IntPtr ctx, IntPtr stream, IntPtr a, IntPtr b, IntPtr bias, IntPtr c,
            int outIsF32, int m, int n, int k, int activation, float actParam);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_bf16gemm_bias_act(IntPtr ctx, IntPtr stream, IntPtr a, IntPtr b, IntPtr bias, IntPtr c,
            int outIsF32, int m, int n, int k, int activation, float actParam);

        // ---- weight-only fp16 GEMM
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_sgemm_f16weight(IntPtr ctx, IntPtr stream, IntPtr a, IntPtr bF16, IntPtr bias, IntPtr c,
            int m, int n, int k, int activation, float actParam);

        // ---- pre-packed weight operand
        [DllImport(Lib, CallingConvention = CC)] internal static extern ulong aidn_mi355_packed_b_bytes(int kind, int k, int n, int transB);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_pack_b(IntPtr ctx, IntPtr stream, int kind, IntPtr b, int k, int n, int transB, IntPtr packed);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_gemm_packed_b(IntPtr ctx, IntPtr stream, int kind, IntPtr a, IntPtr packedB, IntPtr bias, IntPtr c,
            int outIsF32, int m, int n, int k, int transB, int activation, float actParam);

        // ---- 16-bit GEMM, fp32 accumulation
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_hgemm_f32out(IntPtr ctx, IntPtr stream, IntPtr a, IntPtr b, IntPtr c, int m, int n, int k);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_hgemm_f16out(IntPtr ctx, IntPtr stream, IntPtr a, IntPtr b, IntPtr c, int m, int n, int k);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_bf16gemm_f32out(IntPtr ctx, IntPtr stream, IntPtr a, IntPtr b, IntPtr c, int m, int n, int k);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_bf16gemm_bf16out(IntPtr ctx, IntPtr stream, IntPtr a, IntPtr b, IntPtr c, int m, int n, int k);

        // ---- projection + rotary embedding in one call
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_hgemm_rope(IntPtr ctx, IntPtr stream, IntPtr a, IntPtr b, IntPtr c, int m, int n, int k,
            IntPtr cosCache, IntPtr sinCache, int headDim, int ropeCols, int seqLen, int startPosition);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_bf16gemm_rope(IntPtr ctx, IntPtr stream, IntPtr a, IntPtr b, IntPtr c, int m, int n, int k,
            IntPtr cosCache, IntPtr sinCache, int headDim, int ropeCols, int seqLen, int startPosition);

        // ---- storage conversions
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_convert_f32_to_f16(IntPtr ctx, IntPtr stream, IntPtr input, IntPtr output, long n);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_convert_f16_to_f32(IntPtr ctx, IntPtr stream, IntPtr input, IntPtr output, long n);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_convert_f32_to_bf16(IntPtr ctx, IntPtr stream, IntPtr input, IntPtr output, long n);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_convert_bf16_to_f32(IntPtr ctx, IntPtr stream, IntPtr input, IntPtr output, long n);

        // ---- fused scaled-dot-product attention (forward)
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_attn_fwd_f32(IntPtr ctx, IntPtr stream, ref AidnAttnDesc desc,
            IntPtr q, IntPtr k, IntPtr v, IntPtr o, IntPtr lse, IntPtr bias, IntPtr mask, IntPtr weights);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_attn_fwd_f16(IntPtr ctx, IntPtr stream, ref AidnAttnDesc desc,
            IntPtr q, IntPtr k, IntPtr v, IntPtr o, IntPtr lse, IntPtr bias, IntPtr mask, IntPtr weights);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_attn_fwd_bf16(IntPtr ctx, IntPtr stream, ref AidnAttnDesc desc,
            IntPtr q, IntPtr k, IntPtr v, IntPtr o, IntPtr lse, IntPtr bias, IntPtr mask, IntPtr weights);

        // ---- decode attention (Sq == 1)
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_attn_decode_f32(IntPtr ctx, IntPtr stream, ref AidnAttnDesc desc,
            IntPtr q, IntPtr k, IntPtr v, IntPtr o, IntPtr lse, int splits);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_attn_decode_f16(IntPtr ctx, IntPtr stream, ref AidnAttnDesc desc,
            IntPtr q, IntPtr k, IntPtr v, IntPtr o, IntPtr lse, int splits);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_attn_decode_bf16(IntPtr ctx, IntPtr stream, ref AidnAttnDesc desc,
            IntPtr q, IntPtr k, IntPtr v, IntPtr o, IntPtr lse, int splits);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_attn_decode_bf16_noalloc(IntPtr ctx, IntPtr stream, ref AidnAttnDesc desc,
            IntPtr q, IntPtr k, IntPtr v, IntPtr o, IntPtr lse, int splits);

        // ---- attention over a paged K/V cache
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_paged_attn_decode_f32(IntPtr ctx, IntPtr stream, IntPtr q, IntPtr kcache, IntPtr vcache,
            IntPtr blockTable, IntPtr o, int heads, int kvHeads, int headDim, int blockSize, int seqLen, float scale, int splits);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_paged_attn_decode_f16(IntPtr ctx, IntPtr stream, IntPtr q, IntPtr kcache, IntPtr vcache,
            IntPtr blockTable, IntPtr o, int heads, int kvHeads, int headDim, int blockSize, int seqLen, float scale, int splits);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_paged_attn_decode_bf16(IntPtr ctx, IntPtr stream, IntPtr q, IntPtr kcache, IntPtr vcache,
            IntPtr blockTable, IntPtr o, int heads, int kvHeads, int headDim, int blockSize, int seqLen, float scale, int splits);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_paged_attn_prefill_f32(IntPtr ctx, IntPtr stream, IntPtr q, IntPtr kcache, IntPtr vcache,
            IntPtr blockTable, IntPtr o, int heads, int kvHeads, int headDim, int blockSize, int numQueries, int startPos, float scale);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_paged_attn_prefill_f16(IntPtr ctx, IntPtr stream, IntPtr q, IntPtr kcache, IntPtr vcache,
            IntPtr blockTable, IntPtr o, int heads, int kvHeads, int headDim, int blockSize, int numQueries, int startPos, float scale);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_paged_attn_prefill_bf16(IntPtr ctx, IntPtr stream, IntPtr q, IntPtr kcache, IntPtr vcache,
            IntPtr blockTable, IntPtr o, int heads, int kvHeads, int headDim, int blockSize, int numQueries, int startPos, float scale);

        // ---- rotary position embedding, interleaved pairs
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_rope_interleaved_f32(IntPtr ctx, IntPtr stream, IntPtr input, IntPtr cosCache, IntPtr sinCache,
            IntPtr output, long rows, int headDim, int seqLen, int startPosition);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_rope_interleaved_f16(IntPtr ctx, IntPtr stream, IntPtr input, IntPtr cosCache, IntPtr sinCache,
            IntPtr output, long rows, int headDim, int seqLen, int startPosition);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_rope_interleaved_bf16(IntPtr ctx, IntPtr stream, IntPtr input, IntPtr cosCache, IntPtr sinCache,
            IntPtr output, long rows, int headDim, int seqLen, int startPosition);

        // ---- multi-head attention forward
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_mha_fwd_f32(IntPtr ctx, IntPtr stream, IntPtr input, IntPtr wq, IntPtr wk, IntPtr wv,
            IntPtr wo, IntPtr mask, int maskMode, IntPtr output, int batch, int seq, int dModel, int heads);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_mha_fwd_f16(IntPtr ctx, IntPtr stream, IntPtr input, IntPtr wq, IntPtr wk, IntPtr wv,
            IntPtr wo, IntPtr mask, int maskMode, IntPtr output, int batch, int seq, int dModel, int heads);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_mha_fwd_bf16(IntPtr ctx, IntPtr stream, IntPtr input, IntPtr wq, IntPtr wk, IntPtr wv,
            IntPtr wo, IntPtr mask, int maskMode, IntPtr output, int batch, int seq, int dModel, int heads);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_mha_pack_qkv(IntPtr ctx, IntPtr stream, IntPtr wq, IntPtr wk, IntPtr wv, IntPtr packed,
            int dModel, int elemBytes);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_mha_fwd_packed_f32(IntPtr ctx, IntPtr stream, IntPtr input, IntPtr wqkv, IntPtr wo,
            IntPtr mask, int maskMode, IntPtr output, int batch, int seq, int dModel, int heads);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_mha_fwd_packed_f16(IntPtr ctx, IntPtr stream, IntPtr input, IntPtr wqkv, IntPtr wo,
            IntPtr mask, int maskMode, IntPtr output, int batch, int seq, int dModel, int heads);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_mha_fwd_packed_bf16(IntPtr ctx, IntPtr stream, IntPtr input, IntPtr wqkv, IntPtr wo,
            IntPtr mask, int maskMode, IntPtr output, int batch, int seq, int dModel, int heads);

        // ---- test / tuning hooks
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_set_gemm_tile(IntPtr ctx, int tile);
        [DllImport(Lib, CallingConvention = CC)] internal static extern int aidn_mi355_set_attention_fast_path(IntPtr ctx, int enabled);

        private static int s_probe;     // 0 not probed, 1 present, -1 absent

        /// <summary>True when the library loads and answers (probed once); never throws, so that the plain HipBackend keeps
        /// working where the library is not shipped (the pattern of HipBlasNative's availability probe, HipBlasNative.cs:159-170).</summary>
        internal static bool TryLoad()
        {
            if (s_probe != 0) return s_probe > 0;
            try
            {
                s_probe = aidn_mi355_version() != IntPtr.Zero ? 1 : -1;
            }
            catch (DllNotFoundException) { s_probe = -1; }
            catch (EntryPointNotFoundException) { s_probe = -1; }
            catch (BadImageFormatException) { s_probe = -1; }
            return s_probe > 0;
        }

        /// <summary>Turns a non-zero status into the exception the reference's backend would have thrown for the same fault:
        /// ArgumentException for what the native argument checks refuse (the managed guards run first and are more specific),
        /// NotSupportedException for shapes outside the kernels, OutOfMemoryException, InvalidOperationException otherwise
        /// (hipError_t values, the text of HipBackend's CheckHipError).</summary>
        internal static void Check(IntPtr ctx, int status, string op)
        {
            if (status == Ok) return;
            string detail = ctx != IntPtr.Zero ? Marshal.PtrToStringAnsi(aidn_mi355_last_error(ctx)) ?? string.Empty : string.Empty;
            string text = $"{op}: aidotnet_mi355 status {status}" + (detail.Length > 0 ? $" ({detail})" : string.Empty);
            switch (status)
            {
                case ErrInvalidArgument: throw new ArgumentException(text);
                case ErrUnsupported: throw new NotSupportedException(text);
                case ErrOutOfMemory: throw new OutOfMemoryException(text);
                case ErrNoDevice:
                case ErrWorkspace:
                default: throw new InvalidOperationException(text);
            }
        }
    }
}
