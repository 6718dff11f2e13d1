// Host-side launchers shared between the kernel translation units and the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace aidn {

// bias (nullable, N floats added to every row) and act (0 none, 1 ReLU, 2 GELU-tanh, 3 sigmoid, 4 tanh, 5 leaky ReLU with slope
// act_param, 6 swish) form the fused epilogue C = act(alpha A B + beta C + bias)
hipError_t gemm_f32(hipStream_t stream, const float* A, const float* B, float* C, int M, int N, int K,
                    float alpha, float beta, int transB, int batch, long long sA, long long sB, long long sC,
                    int force_tile, const float* bias = nullptr, int act = 0, float act_param = 0.0f, void* workspace = nullptr,
                    const float* Bpre = nullptr, size_t workspace_bytes = 0);
// workspace_bytes: size of `workspace`; a plan whose partials or padded copies would not fit is passed over
// Bpre: B packed once by gemm_f32_pack_b into gemm_f32_packed_b_bytes(N, K, transB) bytes (B itself is then ignored; one batch); the
// workspace must then hold gemm_f32_packed_workspace_bytes(M, N, K, transB) bytes
size_t gemm_f32_packed_b_bytes(int N, int K, int transB);
size_t gemm_f32_packed_workspace_bytes(int M, int N, int K, int transB);
hipError_t gemm_f32_pack_b(hipStream_t stream, const float* B, int K, int N, int transB, void* packed);
// bytes of workspace that let gemm_f32 take its small-M (M <= 8, B [K,N], one batch) or split-K path, and gemm_f32_f16weight its
// small-M path; 0 = not applicable
size_t gemm_f32_workspace_bytes(int M, int N, int K, int transB);
size_t gemm_smallm_workspace_bytes(int M, int N, int K);
// weight-only fp16 GEMM: fp32 A [M,K] x fp16 B [K,N] -> fp32 C (the weights are widened exactly, everything else is fp32)
hipError_t gemm_f32_f16weight(hipStream_t stream, const float* A, const uint16_t* B, float* C, int M, int N, int K,
                              int force_tile, const float* bias = nullptr, int act = 0, float act_param = 0.0f,
                              void* workspace = nullptr, size_t workspace_bytes = 0);
// workspace: gemm_16_workspace_bytes(M, N, K) bytes (0 = none needed); without it the skinny-M path is not taken
size_t gemm_16_workspace_bytes(int M, int N, int K);
// Bpre: B packed once by gemm_16_pack_b into gemm_16_packed_b_bytes(N, K) bytes (B itself is then ignored); the workspace must then
// hold gemm_16_packed_workspace_bytes(M, N, K) bytes
hipError_t gemm_16(hipStream_t stream, int kind, const uint16_t* A, const uint16_t* B, void* C, int out32,
                   int M, int N, int K, int force_tile, void* workspace, size_t workspace_bytes, const float* bias = nullptr, int act = 0,
                   float act_param = 0.0f, const uint16_t* Bpre = nullptr);
// C = A B followed by interleaved RoPE over the first rope.cols columns of C (heads of rope.head_dim elements side by side; row m at
// position rope.start_position + m % rope.seq_len); C has the inputs' type.  Where the product has a summing pass of its own (few
// rows: K ranges side by side) the rotation rides on that pass, otherwise it is a second launch over C.
struct RopeEpilogue { const float* cosc; const float* sinc; int head_dim, cols, seq_len, start_position; };
hipError_t gemm_16_rope(hipStream_t stream, int kind, const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K, int force_tile,
                        void* workspace, size_t workspace_bytes, const RopeEpilogue& rope);
hipError_t rope_cols16(hipStream_t stream, int kind, uint16_t* C, const float* cosc, const float* sinc, int M, int N, int cols, int headDim,
                       int seqLen, int startPosition);
size_t gemm_16_packed_b_bytes(int N, int K);
size_t gemm_16_packed_workspace_bytes(int M, int N, int K);
hipError_t gemm_16_pack_b(hipStream_t stream, const uint16_t* B, int K, int N, void* packed);

// kind: 0 f32->f16, 1 f16->f32, 2 f32->bf16, 3 bf16->f32
hipError_t convert(hipStream_t stream, int kind, const void* in, void* out, long long n);

// interleaved RoPE; kind: 0 fp32, 1 fp16, 2 bf16 (cos / sin caches fp32)
hipError_t rope_interleaved(hipStream_t stream, int kind, const void* in, const float* cosc, const float* sinc, void* out,
                            long long rows, int headDim, int seqLen, int startPosition);

// Attention problem description shared by the prefill and decode launchers (host side).
struct AttnParams {
    const void* q; const void* k; const void* v; void* o;
    float* lse; const float* bias; const float* mask; float* weights;
    int B, H, Hkv, Sq, Sk, D;
    float scale; int causal; int qoff; float softcap; int mask_mode; int out16;
    long long bias_bs;
    long long qs[3], ks[3], vs[3], os[3];   // batch, head, row strides in elements
    // paged K/V (null = contiguous rows): logical key j lives in pool row block_table[j / block_size] * block_size + j % block_size;
    // batch b uses the table at block_table + b * block_table_stride.  The row stride ks[2] / vs[2] is that of the pool.
    const int* block_table = nullptr;
    int block_size = 0;
    long long block_table_stride = 0;
    // 0: every shape takes the general kernel (the direct-to-LDS instances are not used); set per call from the context
    int allow_fast_path = 1;
    // optional scratch of attn_fwd_workspace_bytes() bytes: lets attn_fwd cut the key sequence into ranges when the query tiles
    // alone would leave most of the chip idle
    void* workspace = nullptr;
    size_t workspace_bytes = 0;
};

// Raises a kernel's dynamic shared-memory limit once per device (the attribute belongs to the device's copy of the function).
// Safe to call from several threads: the attribute call is idempotent and the done-mask is atomic.
hipError_t ensure_dynamic_smem(const void* kernel, int bytes, unsigned long long* done_mask);

// kind: 0 fp32, 1 fp16, 2 bf16
hipError_t attn_fwd(hipStream_t stream, int kind, const AttnParams& p);
size_t attn_fwd_workspace_bytes(int kind, const AttnParams& p);

// Decode (Sq == 1).  eff_splits: the split count actually used for `splits` requested (<= 0 = auto).
int attn_decode_splits(int kind, const AttnParams& p, int splits);
// grouped-query decode through the fast prefill kernel (the query heads of a K/V head as the rows of one query tile)
bool attn_group_decode_applies(int kind, const AttnParams& p);
hipError_t attn_group_decode(hipStream_t stream, int kind, const AttnParams& p, int sk, int nsplit, int chunk, float* part);
size_t attn_decode_workspace_bytes(const AttnParams& p, int eff_splits);
hipError_t attn_decode(hipStream_t stream, int kind, const AttnParams& p, int eff_splits, void* workspace);

}  // namespace aidn
