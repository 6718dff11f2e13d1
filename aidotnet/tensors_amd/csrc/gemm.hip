// LDS-staged, double-buffered MFMA GEMM for gfx950: C = alpha * A * op(B) + beta * C,
// row-major, fp32 / fp16 / bf16 inputs with fp32 accumulation.
//
// Replaces, behind the reference's GPU-backend slot, what
// src/AiDotNet.Tensors/Engines/DirectGpu/HIP/HipBackend.cs:1370-1631 (Gemm, MatMulTransposed,
// BatchedGemm) and HipBackend.HalfPrecision.cs:97-150 (Hgemm, GemmFp16In32fOut) do with
// hipBLAS or run-time compiled kernel strings; the arithmetic contract is the CPU path's
// (src/AiDotNet.Tensors/Engines/Simd/SimdGemm.cs:1284-1315, HalfKernels.cs:35-99,
// BFloat16Kernels.cs:144-211): products of the stored values, fp32 accumulation, one
// round-to-nearest-even narrow at the end for 16-bit outputs.
//
// Data movement per workgroup and K-tile (128 bytes of K per row: 64 halves / 32 floats):
//   global --16 B/lane--> registers --(B[K,N]: E x E register transpose)--> LDS [row][k], 144 B
//   row pitch (128 + 16 pad: conflict-free ds_read_b128 / ds_write_b128) --> 16-byte MFMA
//   fragments.  Two LDS stages: the next tile's global loads are issued before the current
//   tile's MFMAs and stored to the other stage after them; one barrier per K-tile.
#include "common.hpp"
#include "launch.hpp"

namespace aidn {

struct GemmArgs {
    const void* A; const void* B; void* C;
    int M, N, K;
    int lda, ldb, ldc;
    long long sA, sB, sC;   // batch strides in elements
    float alpha, beta;
    int tiles_m, tiles_n;
};

constexpr int ROWB = 144;    // LDS row pitch in bytes
constexpr int GROUP_M = 8;   // tile rows walked together so one XCD's L2 sees a compact footprint

// Workgroup id -> (tile row, tile col).  Hardware hands consecutive workgroup ids to the 8
// XCDs round-robin; remap so each XCD owns a contiguous run of logical ids, then walk
// that run in GROUP_M-tall column-major groups.
__device__ __forceinline__ void tile_of_block(int pid, int nblk, int tiles_m, int tiles_n, int& tm, int& tn)
{
    int per = nblk >> 3, rem = nblk & 7;
    int xcd = pid & 7, idx = pid >> 3;
    int logical = (xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per) + idx;
    int width = GROUP_M * tiles_n;
    int group = logical / width;
    int first = group * GROUP_M;
    int gsz = min(tiles_m - first, GROUP_M);
    int in = logical - group * width;
    tm = first + in % gsz;
    tn = in / gsz;
}

template <typename T> struct Raw;
template <> struct Raw<float> { typedef uint32_t type; };
template <> struct Raw<f16_t> { typedef uint16_t type; };
template <> struct Raw<bf16_t> { typedef uint16_t type; };

// 16 bytes = PER16 consecutive elements starting at p, elements at index >= valid read as 0.
template <typename T>
__device__ __forceinline__ u32x4 load16_guarded(const typename Raw<T>::type* p, int valid)
{
    u32x4 v = {0u, 0u, 0u, 0u};
    if constexpr (Elem<T>::BYTES == 4) {
#pragma unroll
        for (int e = 0; e < 4; e++) if (e < valid) v[e] = p[e];
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) if (e < valid) v[e >> 1] |= ((uint32_t)p[e]) << (16 * (e & 1));
    }
    return v;
}

template <typename T, typename OutT, int BM, int BN, int WM, int WN, bool TRANSB, bool VEC, bool CHECK>
__global__ __launch_bounds__(WM * WN * 64) void gemm_kernel(const GemmArgs g)
{
    typedef typename Raw<T>::type raw_t;
    constexpr int E = Elem<T>::PER16;
    constexpr int BK = 8 * E;                  // elements of K per tile (128 bytes)
    constexpr int NT = WM * WN * 64;
    constexpr int WTM = BM / WM, WTN = BN / WN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int UA = (BM * 8 + NT - 1) / NT;                   // 16-byte chunks of A per thread
    constexpr int UBT = (BN * 8 + NT - 1) / NT;                  // same for B stored [N,K]
    constexpr int NBLK = 8 * (BN / E);                           // E x E blocks of B stored [K,N]
    constexpr int UBN = (NBLK + NT - 1) / NT;
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be a multiple of 32x32");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char* As = smem;                          // [2][BM][ROWB]
    unsigned char* Bs = smem + 2 * BM * ROWB;          // [2][BN][ROWB]

    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;

    int tile_m, tile_n;
    tile_of_block(blockIdx.x, gridDim.x, g.tiles_m, g.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const long long bz = blockIdx.z;
    const raw_t* __restrict__ A = (const raw_t*)g.A + bz * g.sA;
    const raw_t* __restrict__ B = (const raw_t*)g.B + bz * g.sB;

    u32x4 ra[UA];
    u32x4 rb[TRANSB ? UBT : UBN * E];

    auto load_tile = [&](int k0) {
        // ---- A (and B when stored [N,K]): 16-byte chunks along K
#pragma unroll
        for (int i = 0; i < UA; i++) {
            int u = t + i * NT;
            int row = u >> 3, ch = u & 7;
            int gm = m0 + row, gk = k0 + ch * E;
            u32x4 v = {0u, 0u, 0u, 0u};
            if ((BM * 8) % NT == 0 || u < BM * 8) {
                const raw_t* p = A + (long long)gm * g.lda + gk;
                if constexpr (!CHECK) v = *(const u32x4*)p;
                else if (gm < g.M && gk < g.K) {
                    if constexpr (VEC) v = *(const u32x4*)p;
                    else v = load16_guarded<T>(p, g.K - gk);
                }
            }
            ra[i] = v;
        }
        if constexpr (TRANSB) {
#pragma unroll
            for (int i = 0; i < UBT; i++) {
                int u = t + i * NT;
                int row = u >> 3, ch = u & 7;
                int gn = n0 + row, gk = k0 + ch * E;
                u32x4 v = {0u, 0u, 0u, 0u};
                if ((BN * 8) % NT == 0 || u < BN * 8) {
                    const raw_t* p = B + (long long)gn * g.ldb + gk;
                    if constexpr (!CHECK) v = *(const u32x4*)p;
                    else if (gn < g.N && gk < g.K) {
                        if constexpr (VEC) v = *(const u32x4*)p;
                        else v = load16_guarded<T>(p, g.K - gk);
                    }
                }
                rb[i] = v;
            }
        } else {
            // ---- B stored [K,N]: E rows of 16 bytes (E consecutive n) per block
#pragma unroll
            for (int i = 0; i < UBN; i++) {
                int u = t + i * NT;
                int kb = u & 7, nb = u >> 3;
                int gn = n0 + nb * E;
#pragma unroll
                for (int r = 0; r < E; r++) {
                    int gk = k0 + kb * E + r;
                    u32x4 v = {0u, 0u, 0u, 0u};
                    if (NBLK % NT == 0 || u < NBLK) {
                        const raw_t* p = B + (long long)gk * g.ldb + gn;
                        if constexpr (!CHECK) v = *(const u32x4*)p;
                        else if (gk < g.K && gn < g.N) {
                            if constexpr (VEC) v = *(const u32x4*)p;
                            else v = load16_guarded<T>(p, g.N - gn);
                        }
                    }
                    rb[i * E + r] = v;
                }
            }
        }
    };

    auto store_tile = [&](int stage) {
        unsigned char* as = As + stage * BM * ROWB;
        unsigned char* bs = Bs + stage * BN * ROWB;
#pragma unroll
        for (int i = 0; i < UA; i++) {
            int u = t + i * NT;
            if ((BM * 8) % NT == 0 || u < BM * 8) *(u32x4*)(as + (u >> 3) * ROWB + (u & 7) * 16) = ra[i];
        }
        if constexpr (TRANSB) {
#pragma unroll
            for (int i = 0; i < UBT; i++) {
                int u = t + i * NT;
                if ((BN * 8) % NT == 0 || u < BN * 8) *(u32x4*)(bs + (u >> 3) * ROWB + (u & 7) * 16) = rb[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < UBN; i++) {
                int u = t + i * NT;
                int kb = u & 7, nb = u >> 3;
                if (NBLK % NT == 0 || u < NBLK) {
                    if constexpr (E == 8) {
                        u32x4 in[8], out[8];
#pragma unroll
                        for (int r = 0; r < 8; r++) in[r] = rb[i * 8 + r];
                        transpose8x8_b16(in, out);
#pragma unroll
                        for (int c = 0; c < 8; c++) *(u32x4*)(bs + (nb * 8 + c) * ROWB + kb * 16) = out[c];
                    } else {
                        u32x4 in[4], out[4];
#pragma unroll
                        for (int r = 0; r < 4; r++) in[r] = rb[i * 4 + r];
                        transpose4x4_b32(in, out);
#pragma unroll
                        for (int c = 0; c < 4; c++) *(u32x4*)(bs + (nb * 4 + c) * ROWB + kb * 16) = out[c];
                    }
                }
            }
        }
    };

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

    const int KT = (g.K + BK - 1) / BK;
    load_tile(0);
    store_tile(0);
    __syncthreads();

    for (int kt = 0; kt < KT; kt++) {
        const int stage = kt & 1;
        if (kt + 1 < KT) load_tile((kt + 1) * BK);
        const unsigned char* as = As + stage * BM * ROWB + (wm * WTM + l32) * ROWB + h * 16;
        const unsigned char* bs = Bs + stage * BN * ROWB + (wn * WTN + l32) * ROWB + h * 16;
#pragma unroll
        for (int s = 0; s < 4; s++) {
            u32x4 fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) fa[i] = *(const u32x4*)(as + i * 32 * ROWB + s * 32);
#pragma unroll
            for (int j = 0; j < TN; j++) fb[j] = *(const u32x4*)(bs + j * 32 * ROWB + s * 32);
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) Mma32<T>::run(acc[i][j], fa[i], fb[j]);
        }
        if (kt + 1 < KT) store_tile(stage ^ 1);
        __syncthreads();
    }

    // ---- epilogue: lane holds column l32 of each 32x32 tile, 16 rows
    typedef typename Raw<OutT>::type out_t;
    out_t* __restrict__ C = (out_t*)g.C + bz * g.sC;
    const bool use_beta = g.beta != 0.0f;
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int col = n0 + wn * WTN + j * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = m0 + wm * WTM + i * 32 + acc_row(r, h);
                if (!CHECK || (row < g.M && col < g.N)) {
                    out_t* p = C + (long long)row * g.ldc + col;
                    float v = g.alpha * acc[i][j][r];
                    if constexpr (Elem<OutT>::BYTES == 4) {
                        if (use_beta) v += g.beta * as_f32(*p);
                        *p = as_u32(v);
                    } else {
                        if (use_beta) v += g.beta * Elem<OutT>::widen(*p);
                        *p = (out_t)Elem<OutT>::narrow(v);
                    }
                }
            }
        }
    }
}

// ------------------------------------------------------------------ host side
template <typename T, typename OutT, int BM, int BN, int WM, int WN, bool TRANSB, bool VEC, bool CHECK>
static hipError_t launch_gemm(GemmArgs g, int batch, hipStream_t stream)
{
    auto kern = gemm_kernel<T, OutT, BM, BN, WM, WN, TRANSB, VEC, CHECK>;
    constexpr int smem = 2 * (BM + BN) * ROWB;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, smem);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    dim3 grid((unsigned)(g.tiles_m * g.tiles_n), 1, (unsigned)batch);
    hipLaunchKernelGGL(kern, grid, dim3(WM * WN * 64), smem, stream, g);
    return hipGetLastError();
}

static bool aligned16(const void* p) { return (((uintptr_t)p) & 15u) == 0; }

// Tile choice: the largest tile that still gives the 256 CUs roughly a full wave of
// workgroups; the unchecked 256x256 instance only for shapes it divides exactly.
template <typename T, typename OutT, bool TRANSB>
static hipError_t dispatch_gemm(const GemmArgs& g, int batch, hipStream_t stream, int force_tile)
{
    constexpr int E = Elem<T>::PER16;
    const bool vec = aligned16(g.A) && aligned16(g.B) && g.lda % E == 0 && g.ldb % E == 0 && g.K % E == 0 &&
                     (TRANSB || g.N % E == 0) && g.sA % E == 0 && g.sB % E == 0;
    auto tiles = [&](int bm, int bn) { return (long long)((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn) * batch; };
    int tile = force_tile;
    if (tile == 0) {
        if constexpr (E == 8 && !TRANSB) {
            if (vec && g.M % 256 == 0 && g.N % 256 == 0 && g.K % 64 == 0 && tiles(256, 256) >= 128) tile = 256;
        }
        if (tile == 0) tile = tiles(128, 128) >= 192 ? 128 : 64;
    }
    if constexpr (E == 8 && !TRANSB) {
        if (tile == 256) {
            if (!(vec && g.M % 256 == 0 && g.N % 256 == 0 && g.K % 64 == 0)) return hipErrorInvalidValue;
            return launch_gemm<T, OutT, 256, 256, 2, 4, TRANSB, true, false>(g, batch, stream);
        }
    }
    if (tile == 128) {
        if (vec) return launch_gemm<T, OutT, 128, 128, 2, 2, TRANSB, true, true>(g, batch, stream);
        return launch_gemm<T, OutT, 128, 128, 2, 2, TRANSB, false, true>(g, batch, stream);
    }
    if (tile == 64) {
        if (vec) return launch_gemm<T, OutT, 64, 64, 2, 2, TRANSB, true, true>(g, batch, stream);
        return launch_gemm<T, OutT, 64, 64, 2, 2, TRANSB, false, true>(g, batch, stream);
    }
    return hipErrorInvalidValue;
}

hipError_t gemm_f32(hipStream_t stream, const float* A, const float* B, float* C, int M, int N, int K,
                    float alpha, float beta, int transB, int batch, long long sA, long long sB, long long sC,
                    int force_tile)
{
    GemmArgs g{A, B, C, M, N, K, K, transB ? K : N, N, sA, sB, sC, alpha, beta, 0, 0};
    if (transB) return dispatch_gemm<float, float, true>(g, batch, stream, force_tile);
    return dispatch_gemm<float, float, false>(g, batch, stream, force_tile);
}

// kind: 0 = fp16, 1 = bf16; out32: C is fp32 (else the same 16-bit type as the inputs)
hipError_t gemm_16(hipStream_t stream, int kind, const uint16_t* A, const uint16_t* B, void* C, int out32,
                   int M, int N, int K, int force_tile)
{
    GemmArgs g{A, B, C, M, N, K, K, N, N, 0, 0, 0, 1.0f, 0.0f, 0, 0};
    if (kind == 0) {
        if (out32) return dispatch_gemm<f16_t, float, false>(g, 1, stream, force_tile);
        return dispatch_gemm<f16_t, f16_t, false>(g, 1, stream, force_tile);
    }
    if (out32) return dispatch_gemm<bf16_t, float, false>(g, 1, stream, force_tile);
    return dispatch_gemm<bf16_t, bf16_t, false>(g, 1, stream, force_tile);
}

}  // namespace aidn
