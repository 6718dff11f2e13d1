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
// Data movement per workgroup and K-tile of the general kernel (128 bytes of K per row, 256 for the 64 x 64 tile):
//   global --16 B/lane--> registers --(B[K,N]: E x E register transpose)--> LDS [row][k], row pitch
//   = row + 16 bytes of padding (conflict-free ds_read_b128 / ds_write_b128) --> 16-byte MFMA
//   fragments.  Two LDS stages: the next tile's global loads are issued at the top of an iteration and
//   stored to the other stage before its last k-step; one barrier per K-tile.
// The 16-bit 256 x 256 kernel further down loads global -> LDS directly; the skinny (M <= 32, 16-bit) and
// small-M (M <= 8, fp32) kernels are bandwidth-bound split-K streams of B.
#include "common.hpp"
#include "launch.hpp"
#include <type_traits>

// This file is compiled three times (the build passes -DAIDN_GEMM_PART=0/1/2) so that its template instances build in
// parallel: part 0 holds the fp32 entry points and everything that exists once, part 1 the fp16 and part 2 the bf16 instances.
#ifndef AIDN_GEMM_PART
#define AIDN_GEMM_PART 0
#endif

namespace aidn {

// f(std::integral_constant<int, I>) for I = BEGIN, BEGIN + STEP, ... < END: a loop the compiler cannot leave rolled (register
// arrays indexed by the loop variable need constant indices)
template <int BEGIN, int END, int STEP, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (BEGIN < END) {
        f(std::integral_constant<int, BEGIN>{});
        static_for<BEGIN + STEP, END, STEP>(f);
    }
}

struct GemmArgs {
    const void* A; const void* B; void* C;
    int M, N, K;
    int lda, ldb, ldc;
    long long sA, sB, sC;   // batch strides in elements
    float alpha, beta;
    int tiles_m, tiles_n;
    // fused epilogue: C = act(alpha * A B + beta * C + bias[col]); bias may be null, act 0 = none
    const float* bias;
    int act;
    float act_param;
    // direct-to-LDS kernels only (the 16 x 16 x 32 one and the instances of the 32 x 32 one with edge handling).  > 0: C has this
    // many columns (fewer than N, the columns past them are padding of B that is computed and dropped) and ldc is any element
    // count, so a row of C may start off a 16-byte boundary
    int c_cols = 0;
};

[[maybe_unused]] static bool aligned16(const void* p) { return (((uintptr_t)p) & 15u) == 0; }

#if AIDN_GEMM_PART == 0
hipError_t ensure_dynamic_smem(const void* kernel, int bytes, unsigned long long* done_mask)
{
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return e;
    const unsigned long long bit = 1ULL << (dev & 63);
    if (__atomic_load_n(done_mask, __ATOMIC_ACQUIRE) & bit) return hipSuccess;
    if (hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes)) return e;
    __atomic_fetch_or(done_mask, bit, __ATOMIC_RELEASE);
    return hipSuccess;
}
#endif

// Pointwise activations of the fused projection epilogues, numbered like the reference's FusedActivationType
// (src/AiDotNet.Tensors/Engines/FusedActivationType.cs:23-70) and computed like its HIP activation kernels
// (src/AiDotNet.Tensors/Engines/DirectGpu/HIP/Kernels/HipActivationKernels.cs:19-70).
__device__ __forceinline__ float apply_activation(float x, int act, float p)
{
    switch (act) {
    case 1: return x < 0.0f ? 0.0f : x;                                                      // ReLU, NaN-preserving form (CpuFusedOperations.cs:1271-1274)
    case 2: return 0.5f * x * (1.0f + tanhf(0.7978845608f * (x + 0.044715f * x * x * x)));   // GELU, tanh form
    case 3: return 1.0f / (1.0f + expf(-x));                                                 // sigmoid
    case 4: return tanhf(x);
    case 5: return x > 0.0f ? x : p * x;                                                     // leaky ReLU, slope p
    case 6: return x / (1.0f + expf(-x));                                                    // swish
    default: return x;
    }
}

// K extent of one tile of the general kernel in 16-byte chunks per row, and the LDS row pitch (one chunk of padding keeps the
// b128 fragment reads conflict-free).  The 64 x 64 tile takes twice the K per barrier: its waves have too little MFMA work
// per tile to hide one barrier every 128 bytes of K.
constexpr int gemm_k_chunks(int bm, int bn) { return bm * bn <= 64 * 64 ? 16 : 8; }
constexpr int gemm_row_pitch(int bm, int bn) { return gemm_k_chunks(bm, bn) * 16 + 16; }
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
    // a whole chunk: one 16-byte load that is only element-aligned (the hardware takes such loads; rows that start off a 16-byte
    // boundary used to be read element by element, ten times slower)
    typedef u32x4 u32x4_a4 __attribute__((aligned(4)));
    typedef u32x4 u32x4_a2 __attribute__((aligned(2)));
    if (valid >= Elem<T>::PER16) {
        if constexpr (Elem<T>::BYTES == 4) return *(const u32x4_a4*)p;
        else return *(const u32x4_a2*)p;
    }
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

// KS = 2: two groups of WM x WN waves work on the same output tile, each on half of the k-steps of every K-tile, and the
// second group's accumulators are added through LDS at the end (for grids too small to give every SIMD two waves).
// Scheduling pattern for one step of straight-line code: NM MFMAs, each followed by its share of ND LDS reads, NV global
// loads and NW LDS writes (in that order of urgency).
template <int NM, int ND, int NV, int NW>
__device__ __forceinline__ void spread_schedule()
{
    constexpr int TOT = ND + NV + NW;
#pragma unroll
    for (int i = 0; i < NM; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
#pragma unroll
        for (int o = i * TOT / NM; o < (i + 1) * TOT / NM; o++) {
            if (o < ND) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            else if (o < ND + NV) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
            else __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
        }
    }
}

// B16 (fp32 kernels only): B holds fp16 weights [K,N]; they are widened to fp32 on the way into LDS, so the product is that
// of the fp32 A with the exactly widened weights, accumulated in fp32 (weight-only fp16 GEMM).
template <typename T, typename OutT, int BM, int BN, int WM, int WN, bool TRANSB, bool VEC, bool CHECK, int KS = 1, bool B16 = false>
__global__ __launch_bounds__(WM * WN * KS * 64) void gemm_kernel(const GemmArgs g)
{
    static_assert(!B16 || (Elem<T>::BYTES == 4 && !TRANSB), "fp16 weights: fp32 kernel, B stored [K,N]");
    typedef typename Raw<T>::type raw_t;
    constexpr int E = Elem<T>::PER16;
    constexpr int KC = gemm_k_chunks(BM, BN);  // 16-byte chunks of K per tile row
    constexpr int BK = KC * E;                 // elements of K per tile
    constexpr int ROWB = gemm_row_pitch(BM, BN);
    constexpr int NT = WM * WN * KS * 64;
    constexpr int SPG = KC / 2 / KS;                // fragment steps of a K-tile per wave group
    static_assert(KS == 1 || KS == 2, "KS must be 1 or 2");
    constexpr int WTM = BM / WM, WTN = BN / WN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int UA = (BM * KC + NT - 1) / NT;                   // 16-byte chunks of A per thread
    constexpr int UBT = (BN * KC + NT - 1) / NT;                  // same for B stored [N,K]
    constexpr int NBLK = KC * (BN / E);                           // E x E blocks of B stored [K,N]
    constexpr int UBN = (NBLK + NT - 1) / NT;
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be a multiple of 32x32");

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char* As = smem;                          // [2][BM][ROWB]
    unsigned char* Bs = smem + 2 * BM * ROWB;          // [2][BN][ROWB]

    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    const int kgrp = wave / (WM * WN), wq = wave - kgrp * (WM * WN);
    const int wm = wq / WN, wn = wq % WN;

    int tile_m, tile_n;
    tile_of_block(blockIdx.x, gridDim.x, g.tiles_m, g.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const long long bz = blockIdx.z;
    const raw_t* __restrict__ A = (const raw_t*)g.A + bz * g.sA;
    const raw_t* __restrict__ B = (const raw_t*)g.B + bz * g.sB;

    // Global loads run two tiles ahead where the registers allow it (tile t travels in register set t & 1 and has two
    // iterations to arrive from memory: what a small problem with one workgroup per CU needs), otherwise one tile ahead.
    constexpr bool AHEAD2 = BM * BN <= 64 * 64;
    constexpr int NSETS = AHEAD2 ? 2 : 1;
    u32x4 ra2[NSETS][UA];
    u32x4 rb2[NSETS][TRANSB ? UBT : UBN * E];

    auto load_tile = [&](int k0, auto setc) {
        auto& ra = ra2[decltype(setc)::value];
        auto& rb = rb2[decltype(setc)::value];
        // ---- A (and B when stored [N,K]): 16-byte chunks along K
#pragma unroll
        for (int i = 0; i < UA; i++) {
            int u = t + i * NT;
            int row = u / KC, ch = u % KC;
            int gm = m0 + row, gk = k0 + ch * E;
            u32x4 v = {0u, 0u, 0u, 0u};
            if ((BM * KC) % NT == 0 || u < BM * KC) {
                const raw_t* p = A + (long long)(CHECK ? gm : min(gm, g.M - 1)) * g.lda + gk;
                if constexpr (!CHECK) v = *(const u32x4*)p;       // rows past the end repeat the last one (never stored)
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
                int row = u / KC, ch = u % KC;
                int gn = n0 + row, gk = k0 + ch * E;
                u32x4 v = {0u, 0u, 0u, 0u};
                if ((BN * KC) % NT == 0 || u < BN * KC) {
                    const raw_t* p = B + (long long)(CHECK ? gn : min(gn, g.N - 1)) * g.ldb + gk;
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
                int kb = u % KC, nb = u / KC;
                int gn = n0 + nb * E;
#pragma unroll
                for (int r = 0; r < E; r++) {
                    int gk = k0 + kb * E + r;
                    u32x4 v = {0u, 0u, 0u, 0u};
                    if (NBLK % NT == 0 || u < NBLK) {
                        if constexpr (B16) {
                            const uint16_t* p = (const uint16_t*)g.B + bz * g.sB + (long long)gk * g.ldb + gn;
                            if (gk < g.K && gn < g.N) {
                                if (VEC && gn + 4 <= g.N) {
                                    u32x2 w = *(const u32x2*)p;
                                    v = u32x4{as_u32(f16_bits_to_float(w[0] & 0xFFFFu)), as_u32(f16_bits_to_float(w[0] >> 16)),
                                              as_u32(f16_bits_to_float(w[1] & 0xFFFFu)), as_u32(f16_bits_to_float(w[1] >> 16))};
                                } else {
#pragma unroll
                                    for (int e = 0; e < 4; e++) if (gn + e < g.N) v[e] = as_u32(f16_bits_to_float(p[e]));
                                }
                            }
                        } else {
                        const raw_t* p = B + (long long)gk * g.ldb + (CHECK ? gn : min(gn, g.N - E));
                        if constexpr (!CHECK) v = *(const u32x4*)p;   // column blocks past the end repeat the last one
                        else if (gk < g.K && gn < g.N) {
                            if constexpr (VEC) v = *(const u32x4*)p;
                            else v = load16_guarded<T>(p, g.N - gn);
                        }
                        }
                    }
                    rb[i * E + r] = v;
                }
            }
        }
    };

    auto store_tile = [&](int stage, auto setc) {
        auto& ra = ra2[decltype(setc)::value];
        auto& rb = rb2[decltype(setc)::value];
        unsigned char* as = As + stage * BM * ROWB;
        unsigned char* bs = Bs + stage * BN * ROWB;
#pragma unroll
        for (int i = 0; i < UA; i++) {
            int u = t + i * NT;
            if ((BM * KC) % NT == 0 || u < BM * KC) *(u32x4*)(as + (u / KC) * ROWB + (u % KC) * 16) = ra[i];
        }
        if constexpr (TRANSB) {
#pragma unroll
            for (int i = 0; i < UBT; i++) {
                int u = t + i * NT;
                if ((BN * KC) % NT == 0 || u < BN * KC) *(u32x4*)(bs + (u / KC) * ROWB + (u % KC) * 16) = rb[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < UBN; i++) {
                int u = t + i * NT;
                int kb = u % KC, nb = u / KC;
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
                        for (int r = 0; r < 4; r++) {
                            in[r] = rb[i * 4 + r];
                            // the renaming moves belong here, not behind the global loads (where they would wait for them)
                            asm volatile("" : "+v"(in[r]));
                        }
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
    typedef std::integral_constant<int, 0> Set0;
    typedef std::integral_constant<int, 1> Set1;
    load_tile(0, Set0{});
    store_tile(0, Set0{});
    if constexpr (AHEAD2) {
        if (!CHECK || KT > 1) load_tile(min(1, KT - 1) * BK, Set1{});
    }
    __syncthreads();

    // Fragments are double-buffered in registers: the LDS reads of step s+1 are in flight during the MFMAs of step s.
    // Tile kt+1 is published (register -> LDS stores, barrier) BEFORE the last step of tile kt, and its first fragments are
    // read right after the barrier, so the barrier wait and the LDS latency are covered by that step's MFMAs.
    const int frag_off = (wm * WTM + l32) * ROWB + h * 16 + kgrp * SPG * 32;
    const int frag_off_b = (wn * WTN + l32) * ROWB + h * 16 + kgrp * SPG * 32;
    u32x4 fa[2][TM], fb[2][TN];
    auto read_frags = [&](int stage, int step, int buf) {
        const unsigned char* as = As + stage * BM * ROWB + frag_off + step * 32;
        const unsigned char* bs = Bs + stage * BN * ROWB + frag_off_b + step * 32;
#pragma unroll
        for (int i = 0; i < TM; i++) fa[buf][i] = *(const u32x4*)(as + i * 32 * ROWB);
#pragma unroll
        for (int j = 0; j < TN; j++) fb[buf][j] = *(const u32x4*)(bs + j * 32 * ROWB);
    };
    // iteration kt works on LDS stage kt & 1 = SET, requests tile kt+2 into register set SET (free: tile kt was stored one
    // iteration ago) and publishes tile kt+1 from the other set; with one set it requests tile kt+1 and publishes it
    auto iteration = [&](int kt, int SET, auto intoc, auto otherc) {
        typedef decltype(intoc) Into;
        typedef decltype(otherc) Other;
        // The unchecked instance has no branch in the loop body (past the end it fetches the last tile once more and
        // publishes it to the unused stage), so loads, LDS traffic and MFMAs of one iteration can be interleaved freely.
        const bool more = !CHECK || kt + 1 < KT;
        if constexpr (!CHECK) load_tile(min(kt + NSETS, KT - 1) * BK, Into{});
        else if (kt + NSETS < KT) load_tile((kt + NSETS) * BK, Into{});
#pragma unroll
        for (int s = 0; s < SPG; s++) {
            if (s < SPG - 1) read_frags(SET, s + 1, (s + 1) & 1);
            else {
                __builtin_amdgcn_sched_barrier(0);      // keep the MFMAs of the last step below the barrier
                if (more) store_tile(SET ^ 1, Other{});
                __syncthreads();
                if (more) read_frags(SET ^ 1, 0, SPG & 1);
            }
            __builtin_amdgcn_sched_barrier(0);          // fragment reads of the next step are issued before this step's MFMAs
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) Mma32<T>::run(acc[i][j], fa[s & 1][i], fb[s & 1][j]);
        }
    };
    // Unchecked instance: one iteration is straight-line code, and the order of its instructions is given explicitly: every
    // MFMA is followed by its share of the step's other memory instructions (next fragments, the global loads in the first
    // step, the LDS stores of the next tile in the last step before the barrier), so the matrix pipe never waits behind a
    // burst of them.
    auto mfma_step = [&](int s) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) Mma32<T>::run(acc[i][j], fa[s & 1][i], fb[s & 1][j]);
    };
    auto iteration_il = [&](int kt, int SET, auto intoc, auto otherc) {
        typedef decltype(intoc) Into;
        typedef decltype(otherc) Other;
        constexpr int NM = TM * TN * (E == 4 ? 4 : 1);          // MFMAs per step
        constexpr int NL = UA + (TRANSB ? UBT : UBN * E);       // global loads = LDS stores per tile and thread
        constexpr int NR = TM + TN;                             // fragment reads per step
        load_tile(min(kt + NSETS, KT - 1) * BK, Into{});
#pragma unroll
        for (int s = 0; s < SPG - 1; s++) {
            read_frags(SET, s + 1, (s + 1) & 1);
            if (s == SPG - 2) store_tile(SET ^ 1, Other{});
            mfma_step(s);
            if (s == 0 && s == SPG - 2) spread_schedule<NM, NR, NL, NL>();
            else if (s == 0) spread_schedule<NM, NR, NL, 0>();
            else if (s == SPG - 2) spread_schedule<NM, NR, 0, NL>();
            else spread_schedule<NM, NR, 0, 0>();
            __builtin_amdgcn_sched_barrier(0);
        }
        __syncthreads();
        read_frags(SET ^ 1, 0, SPG & 1);
        mfma_step(SPG - 1);
        spread_schedule<NM, NR, 0, 0>();
        __builtin_amdgcn_sched_barrier(0);
    };
    read_frags(0, 0, 0);
    if constexpr (!CHECK && AHEAD2) {
        for (int kt = 0; kt < KT; kt += 2) {
            iteration_il(kt, 0, Set0{}, Set1{});
            if (kt + 1 < KT) iteration_il(kt + 1, 1, Set1{}, Set0{});
        }
    } else if constexpr (!CHECK) {
        for (int kt = 0; kt < KT; kt++) iteration_il(kt, kt & 1, Set0{}, Set0{});
    } else if constexpr (AHEAD2) {
        for (int kt = 0; kt < KT; kt += 2) {
            iteration(kt, 0, Set0{}, Set1{});
            if (kt + 1 < KT) iteration(kt + 1, 1, Set1{}, Set0{});
        }
    } else {
        for (int kt = 0; kt < KT; kt++) iteration(kt, kt & 1, Set0{}, Set0{});
    }

    if constexpr (KS == 2) {
        // second wave group hands its partial sums over through LDS (the tile stages are free after the last barrier)
        float* xs = (float*)smem;
        if (kgrp == 1) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
#pragma unroll
                    for (int r = 0; r < 16; r++) xs[((wq * TM + i) * TN + j) * 1024 + r * 64 + lane] = acc[i][j][r];
        }
        __syncthreads();
        if (kgrp == 1) return;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] += xs[((wq * TM + i) * TN + j) * 1024 + r * 64 + lane];
    }

    // ---- epilogue: lane holds column l32 of each 32x32 tile, 16 rows
    typedef typename Raw<OutT>::type out_t;
    out_t* __restrict__ C = (out_t*)g.C + bz * g.sC;
    const bool use_beta = g.beta != 0.0f;
    const bool fused = g.bias != nullptr || g.act != 0;
    auto store_all = [&](auto fused_c) {
        constexpr bool FUSED = decltype(fused_c)::value;
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int j = 0; j < TN; j++) {
                const int col = n0 + wn * WTN + j * 32 + l32;
                float bias = 0.0f;
                if constexpr (FUSED) bias = (g.bias && col < g.N) ? g.bias[col] : 0.0f;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int row = m0 + wm * WTM + i * 32 + acc_row(r, h);
                    if (row < g.M && col < g.N) {
                        out_t* p = C + (long long)row * g.ldc + col;
                        float v = g.alpha * acc[i][j][r];
                        if constexpr (Elem<OutT>::BYTES == 4) {
                            if (use_beta) v += g.beta * as_f32(*p);
                            if constexpr (FUSED) v = apply_activation(v + bias, g.act, g.act_param);
                            *p = as_u32(v);
                        } else {
                            if (use_beta) v += g.beta * Elem<OutT>::widen(*p);
                            if constexpr (FUSED) v = apply_activation(v + bias, g.act, g.act_param);
                            *p = (out_t)Elem<OutT>::narrow(v);
                        }
                    }
                }
            }
        }
    };
    if (fused) store_all(std::true_type{});
    else store_all(std::false_type{});
}

// ---------------------------------------------------------------------------------------------
// Large-tile fast path for 16-bit inputs, B stored [K,N]: 256 x 256 x 64 tile, 8 waves (2 x 4, wave tile
// 128 x 64).  Requires M % 256 == 0, N % 256 == 0, K % 64 == 0 and 16-byte aligned rows.
//   * global -> LDS by the gfx950 direct load (global_load_lds_dwordx4): no staging registers, no
//     ds_write, no register transposes.  One wave-load moves 64 lanes x 16 B into 1 KiB of contiguous LDS,
//     so bank-conflict avoidance is done by choosing WHICH global chunk a lane fetches (XOR swizzle):
//       A tile [256 rows][128 B]: 16-byte chunk c of row r lives at chunk position c ^ ((r >> 1) & 7)
//       B tile [64 k][512 B]    : 16-byte chunk c of row k lives at chunk position c ^ ((k & 3) << 2)
//   * B fragments come out of the [k][n] tile with the transposing LDS read ds_read_b64_tr_b16: within
//     a 16-lane group, lane i receives element (i % 4) of the 8 bytes addressed by lane 4 m + i / 4,
//     for m = 0..3; lanes address B[k0 + j/4][n0 + 4 (j%4)] and receive B[k0 .. k0+3][n0 + i].
//   * the DMA is issued through inline asm: with the builtin the compiler orders every later LDS read
//     that may alias the destination behind s_waitcnt vmcnt(0), which serialises load latency and MFMA.
//     Completion is waited for explicitly (vmcnt(0) + workgroup barrier) before a stage is read.
typedef short s16x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void dma16_to_lds(const void* gptr, void* lds_dst_wave_uniform)
{
    uint32_t l = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)lds_dst_wave_uniform);
    l = __builtin_amdgcn_readfirstlane(l);
    // M0 carries the LDS base of the wave's 1 KiB destination; nothing else in these kernels uses M0
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(l), "v"(gptr));
}

// same for data that is read once per launch (a streamed weight matrix): non-temporal, so that it does not displace what the
// caches hold for reuse (a plain read loop reaches 6.0-6.2 TB/s on this part, a non-temporal one 6.9-7.0 TB/s)
__device__ __forceinline__ void dma16_to_lds_stream(const void* gptr, void* lds_dst_wave_uniform)
{
    uint32_t l = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)lds_dst_wave_uniform);
    l = __builtin_amdgcn_readfirstlane(l);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off nt" ::"s"(l), "v"(gptr));
}

// same, source = wave-uniform base (scalar register pair) + per-lane unsigned 32-bit byte offset, destination given as the LDS
// byte address
__device__ __forceinline__ void dma16_base(const void* base_uniform, uint32_t lane_off, uint32_t lds_dst)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_dst), "v"(lane_off), "s"(base_uniform) : "memory");
}

// EDGE: M, N and K need not be multiples of the tile (N and K still multiples of 8): loads of rows / column chunks past the
// end are redirected to the last valid one (their products land in accumulator elements that are never stored), the stores
// are guarded, and in the last, partial K-tile every 16-byte chunk at or past K is fetched from a block of zeros instead.
__device__ __attribute__((aligned(16))) const uint32_t g_zero_chunk[4] = {0u, 0u, 0u, 0u};

// direct global -> LDS load with a full per-lane address (the form for lanes that do not share a base)
__device__ __forceinline__ void dma16_addr(const void* gptr, uint32_t lds_dst)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_dst), "v"(gptr) : "memory");
}

// TILE = 256: 8 waves (2 x 4), wave tile 128 x 64, one workgroup per CU.  TILE = 128: 4 waves (2 x 2), wave tile 64 x 64, two
// workgroups per CU (for problems with too few 256 x 256 tiles to occupy the chip).
// TRANSB: B is stored [N,K]; its tile is then loaded and read exactly like the A tile (rows of 128 bytes of K, b128 fragments).
// KSW = 2 (fp32, 64 x 64 tile, whole tiles): eight waves, two groups of four that take half of the k-steps of every K-tile each and are
// summed through LDS at the end (group 0 + group 1, a fixed order).  With about one such tile per CU the four-wave form runs one wave
// per SIMD, which has nothing to switch to while it issues loads or waits at the tile barrier (matrix pipe 69 % busy at 1024^3).
template <typename T, typename OutT, bool EDGE = false, int TILE = 256, bool TRANSB = false, int KSW = 1>
__global__ __launch_bounds__((TILE == 256 ? 512 : 256) * KSW, TILE == 256 ? 1 : 2) void gemm_dl_kernel(const GemmArgs g)
{
    constexpr int E = Elem<T>::PER16, EB = Elem<T>::BYTES;
    static_assert(TILE == 256 || TILE == 128 || TILE == 64, "tile edge");
    static_assert(KSW == 1 || (KSW == 2 && TILE == 64 && EB == 4 && !EDGE && !TRANSB), "the split form exists for the fp32 64 x 64 tile");
    constexpr int WM = 2, WN = TILE == 256 ? 4 : 2;
    constexpr int BM = TILE, BN = TILE, BK = 128 / EB;          // 128 bytes of K per tile row: 64 halves / 32 floats
    constexpr int WTM = BM / WM, WTN = BN / WN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int BROW = BN * EB;                 // bytes of one k-row of the B tile
    constexpr int ABYTES = BM * 128, BBYTES = BK * BROW, STAGE = ABYTES + BBYTES;
    constexpr int NWAVE = WM * WN * KSW;
    constexpr int LA = BM / 8 / NWAVE, LB = LA;       // 1 KiB wave-loads per wave per tile (4 + 4; 2 + 2 for the 64 x 64 tile, 1 + 1 in its split form)
    constexpr int RPL = 1024 / BROW;              // k-rows of B per wave-load
    constexpr int LPR = 64 / RPL;                 // lanes (16-byte chunks) per B row
    static_assert(BK * BROW / 1024 == LB * NWAVE && BN / 8 == LB * NWAVE && (LA % 2 == 0 || KSW == 2), "B tile = as many wave-loads as the A tile");

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;                 // wave: index among all waves (partition of the loads)
    const int l32 = lane & 31, h = lane >> 5;
    const int kgrp = KSW == 1 ? 0 : wave / (WM * WN);      // k-step group
    const int wq = KSW == 1 ? wave : wave % (WM * WN);
    const int wm = wq / WN, wn = wq % WN;
    int tile_m, tile_n;
    tile_of_block(blockIdx.x, gridDim.x, g.tiles_m, g.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const long long bz = blockIdx.z;                                         // batch index (strides in elements)
    const unsigned char* __restrict__ A = (const unsigned char*)g.A + bz * g.sA * EB;
    const unsigned char* __restrict__ B = (const unsigned char*)g.B + bz * g.sB * EB;

    // Chunk swizzle of the B tile (which 16-byte chunk position of its LDS row a chunk of k-row `row` occupies):
    //   16-bit: c ^ ((row & 3) << 2)  -- the four rows one transposing read touches go to different bank groups (rows of 256
    //           bytes and more; 128-byte rows, which alternate between the bank halves by themselves: c ^ (((row >> 1) & 1) << 2));
    //   fp32:   c ^ (((row >> 2) & 1) << 3)  -- the two lane halves of a b32 fragment read (rows 4 apart) use different bank halves.
    auto b_swz = [](int row) -> int {
        return E == 8 ? (BROW >= 256 ? ((row & 3) << 2) : (((row >> 1) & 1) << 2)) : (((row >> 2) & 1) << 3);
    };

    // Sources of this wave's loads: a wave-uniform base (scalar registers, advanced per tile by scalar adds) plus a per-lane
    // 32-bit byte offset that never changes, so issuing a load costs no vector instruction.  Wave-load w = 4 wave + i covers
    // A rows 8w .. 8w+7 resp. B k-rows RPL w .. RPL w + RPL-1.
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)smem);
    uint32_t a_lane_off[EDGE ? LA : 2], b_lane_off[LB];
#pragma unroll
    for (int par = 0; par < 2; par++) {
        const int ra = lane >> 3, pos_a = lane & 7;           // row inside the wave-load, 16-byte chunk
        // (the swizzle of a row is ((row >> 1) & 7) with row = 8 (LA wave + i) + ra: only the parity of LA wave + i enters)
        if constexpr (!EDGE) a_lane_off[par] = (uint32_t)(ra * g.lda + (pos_a ^ ((4 * par + (ra >> 1)) & 7)) * E) * (uint32_t)EB;
    }
#pragma unroll
    for (int i = 0; i < LB; i++) {
        if constexpr (TRANSB) {
            const int rn = lane >> 3, pos = lane & 7;             // like A: wave-load w covers tile rows (n) 8w .. 8w+7
            int row = 8 * (LB * wave + i) + rn;
            const int sw = (row >> 1) & 7;
            if constexpr (EDGE) row = min(row, g.N - 1 - n0);
            else row = rn;                                        // relative to the wave-load's first row (scalar base)
            b_lane_off[i] = (uint32_t)(row * g.ldb + (pos ^ sw) * E) * (uint32_t)EB;
        } else {
            const int rb = lane / LPR, pos_b = lane % LPR;
            int chunk = pos_b ^ b_swz(RPL * (LB * wave + i) + rb);
            if constexpr (EDGE) chunk = min(chunk, (g.N - n0) / E - 1);      // N % E == 0 and n0 < N: at least one chunk
            b_lane_off[i] = (uint32_t)(rb * g.ldb + chunk * E) * (uint32_t)EB;
        }
    }
    if constexpr (EDGE) {
#pragma unroll
        for (int i = 0; i < LA; i++) {
            const int ra = lane >> 3, pos_a = lane & 7;
            const int row = min(8 * (LA * wave + i) + ra, g.M - 1 - m0);      // source row inside the tile (m0 < M)
            a_lane_off[i] = (uint32_t)(row * g.lda + (pos_a ^ ((4 * (i & 1) + (ra >> 1)) & 7)) * E) * (uint32_t)EB;
        }
    }
    // (EDGE: the A offsets are relative to the tile's first row, since a clamped row may lie before the wave's own rows)
    const unsigned char* a_base = A + (long long)(m0 + (EDGE ? 0 : 8 * LA * wave_s)) * g.lda * EB;
    const unsigned char* b_base = TRANSB ? B + (long long)(n0 + (EDGE ? 0 : 8 * LB * wave_s)) * g.ldb * EB
                                         : B + ((long long)(RPL * LB * wave_s) * g.ldb + n0) * EB;
    // bytes between consecutive wave-loads
    const long long a_step = 8LL * g.lda * EB, b_step = TRANSB ? (EDGE ? 0LL : 8LL * g.ldb * EB) : (long long)RPL * g.ldb * EB;
    const int KT = (g.K + BK - 1) / BK;
    const int ktail = EDGE ? g.K - (KT - 1) * BK : BK;                        // k-rows of the last tile (BK when K % BK == 0)
    auto issue_loads = [&](int kt, int stage) {
        const uint32_t as = lds0 + stage * STAGE + wave_s * (LA * 1024);
        const uint32_t bs = lds0 + stage * STAGE + ABYTES + wave_s * (LB * 1024);
        const unsigned char* a_src = a_base + (long long)kt * 128;
        const unsigned char* b_src = TRANSB ? b_base + (long long)kt * 128 : b_base + (long long)kt * BK * g.ldb * EB;
        if constexpr (EDGE) {
            if (kt == KT - 1 && ktail < BK) {
                // partial last tile: chunks at or past K come from the zero block (a product with zero adds nothing)
#pragma unroll
                for (int i = 0; i < LA; i++) {
                    const int ra = lane >> 3, pos_a = lane & 7;
                    const int chunk = pos_a ^ ((4 * (i & 1) + (ra >> 1)) & 7);               // the chunk this lane fetches
                    const void* src = chunk * E < ktail ? (const void*)(a_src + a_lane_off[i]) : (const void*)g_zero_chunk;
                    dma16_addr(src, as + i * 1024);
                }
#pragma unroll
                for (int i = 0; i < LB; i++) {
                    bool valid;
                    if constexpr (TRANSB) {
                        const int rn = lane >> 3, pos = lane & 7;
                        valid = (pos ^ (((8 * (LB * wave + i) + rn) >> 1) & 7)) * E < ktail;  // the chunk of K this lane fetches
                    } else {
                        valid = RPL * (LB * wave + i) + lane / LPR < ktail;                  // k-row inside the tile
                    }
                    const void* src = valid ? (const void*)(b_src + i * b_step + b_lane_off[i]) : (const void*)g_zero_chunk;
                    dma16_addr(src, bs + i * 1024);
                }
                return;
            }
        }
#pragma unroll
        for (int i = 0; i < LA; i++) {
            if constexpr (EDGE) dma16_base(a_src, a_lane_off[i], as + i * 1024);
            else dma16_base(a_src + i * a_step, a_lane_off[LA % 2 == 0 ? (i & 1) : ((wave + i) & 1)], as + i * 1024);
        }
#pragma unroll
        for (int i = 0; i < LB; i++) dma16_base(b_src + i * b_step, b_lane_off[i], bs + i * 1024);
    };

    // per-lane LDS read offsets
    int a_off[TM], a_sw[TM];
#pragma unroll
    for (int i = 0; i < TM; i++) {
        int row = wm * WTM + i * 32 + l32;
        a_off[i] = row * 128;
        a_sw[i] = ((row >> 1) & 7) ^ (KSW == 2 ? 4 * kgrp : 0);      // group g reads k-steps 2 g and 2 g + 1: chunk (2 (2 g + u) + h) ^ sw
    }
    // 16-bit B fragments (transposing reads): lane j of a 16-lane group addresses k-row (base + j / 4), 8 bytes
    const int jl = lane & 15;
    const int b_rowl = 8 * h + (jl >> 2);                     // + 16 s + 4 q
    const int b_half = (jl & 1) * 8;
    int b_chunk[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) b_chunk[j] = (wn * WTN + j * 32 + 16 * ((lane >> 4) & 1) + 4 * (jl & 3)) >> 3;
    // fp32 B fragments (b32 reads): lane (h, l32) reads column l32 of k-rows 8 s + 4 h + (0..3); (row >> 2) & 1 == h there
    int b_col32[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) {
        const int col = wn * WTN + j * 32 + l32;
        b_col32[j] = (((col >> 2) ^ (h << 3)) << 4) + (col & 3) * 4 + 4 * h * BROW + (KSW == 2 ? 16 * kgrp * BROW : 0);
    }

    int bt_off[TN], bt_sw[TN];                               // B stored [N,K]: like the A fragments
#pragma unroll
    for (int j = 0; j < TN; j++) {
        int row = wn * WTN + j * 32 + l32;
        bt_off[j] = row * 128;
        bt_sw[j] = (row >> 1) & 7;
    }

    auto read_frags = [&](const unsigned char* as, const unsigned char* bs, int s, u32x4 (&fa)[TM], u32x4 (&fb)[TN]) {
#pragma unroll
        for (int i = 0; i < TM; i++) fa[i] = *(const u32x4*)(as + a_off[i] + (((2 * s + h) ^ a_sw[i]) << 4));
#pragma unroll
        for (int j = 0; j < TN; j++) {
            if constexpr (TRANSB) {
                fb[j] = *(const u32x4*)(bs + bt_off[j] + (((2 * s + h) ^ bt_sw[j]) << 4));
            } else if constexpr (E == 4) {
#pragma unroll
                for (int q = 0; q < 4; q++) fb[j][q] = *(const uint32_t*)(bs + (8 * s + q) * BROW + b_col32[j]);
            } else {
#pragma unroll
                for (int q = 0; q < 2; q++) {
                    int row = 16 * s + 4 * q + b_rowl;
                    int pos = b_chunk[j] ^ b_swz(row);
                    s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) s16x4*)(bs + row * BROW + pos * 16 + b_half));
                    u32x2 w = __builtin_bit_cast(u32x2, v);
                    fb[j][2 * q] = w[0];
                    fb[j][2 * q + 1] = w[1];
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

    issue_loads(0, 0);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();

    // Software pipeline: the fragments of k-step s+1 are read from LDS before the MFMAs of step s are issued, so the
    // LDS latency runs under 8 MFMAs; the barrier that publishes tile kt+1 sits before the MFMAs of the last step, and the
    // first fragments of tile kt+1 are read there too.  sched_barrier pins this order (the scheduler otherwise sinks
    // the reads next to their use to save registers, which exposes the LDS latency every few MFMAs).
    u32x4 fa[2][TM], fb[2][TN];
    read_frags(smem, smem + ABYTES, 0, fa[0], fb[0]);
    for (int kt = 0; kt < KT; kt++) {
        const int stage = kt & 1;
        const unsigned char* as = smem + stage * STAGE;
        const unsigned char* bs = as + ABYTES;
        // the other stage was last read before the barrier inside the previous iteration
        if (kt + 1 < KT) issue_loads(kt + 1, stage ^ 1);
#pragma unroll
        for (int s = 0; s < 4 / KSW; s++) {        // (split form: the group's two k-steps; the fragment bases carry the group's offset)
            if (s < 4 / KSW - 1) {
                read_frags(as, bs, s + 1, fa[(s + 1) & 1], fb[(s + 1) & 1]);
            } else {
                __builtin_amdgcn_s_waitcnt(0);      // this wave's DMA has landed and its LDS reads of this tile are done ...
                __syncthreads();                    // ... and so have everyone else's
                if (kt + 1 < KT) {
                    const unsigned char* an = smem + (stage ^ 1) * STAGE;
                    read_frags(an, an + ABYTES, 0, fa[0], fb[0]);
                }
            }
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) Mma32<T>::run(acc[i][j], fa[s & 1][i], fb[s & 1][j]);
            // the next step's fragment reads go behind the first half of this step's MFMAs (two each), so the matrix pipe does
            // not wait behind a burst of reads and the last read still has half a step to complete
            constexpr int NMF = TM * TN * (E == 4 ? 4 : 1);             // MFMA instructions per step
            spread_schedule<NMF / 2, TM + (TRANSB ? 1 : E == 4 ? 4 : 2) * TN, 0, 0>();
            __builtin_amdgcn_sched_group_barrier(0x008, NMF - NMF / 2, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    }

    if constexpr (KSW == 2) {
        // nobody reads the tile ring after the last barrier: group 1 parks its accumulators there, group 0 adds them to its own
        float* red = (float*)smem;
        if (kgrp == 1) {
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
#pragma unroll
                    for (int r = 0; r < 16; r++) red[(((wq * TM + i) * TN + j) * 16 + r) * 64 + lane] = acc[i][j][r];
        }
        __syncthreads();
        if (kgrp == 1) return;
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] += red[(((wq * TM + i) * TN + j) * 16 + r) * 64 + lane];
    }
    typedef typename Raw<OutT>::type out_t;
    out_t* __restrict__ C = (out_t*)g.C + bz * g.sC;
    const bool fused = g.bias != nullptr || g.act != 0;
    if (Elem<OutT>::BYTES == 4 && (g.alpha != 1.0f || g.beta != 0.0f)) {
        // C = act(alpha A B + beta C + bias), fp32 output only: the uncommon form, kept apart so the plain stores below stay lean
#pragma unroll 1
        for (int ij = 0; ij < TM * TN; ij++) {
            const int i = ij / TN, j = ij - i * TN;
            const int col = n0 + wn * WTN + j * 32 + l32;
            if (EDGE && col >= (g.c_cols > 0 ? g.c_cols : g.N)) continue;
            const float bias = g.bias ? g.bias[col] : 0.0f;
            f32x16 v = acc[0][0];
#pragma unroll
            for (int ii = 0; ii < TM; ii++)
#pragma unroll
                for (int jj = 0; jj < TN; jj++) if (ii == i && jj == j) v = acc[ii][jj];
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = m0 + wm * WTM + i * 32 + acc_row(r, h);
                if (EDGE && row >= g.M) continue;
                out_t* p = C + (long long)row * g.ldc + col;
                float x = g.alpha * v[r];
                if (g.beta != 0.0f) {
                    if constexpr (Elem<OutT>::BYTES == 4) x += g.beta * as_f32(*p);
                    else x += g.beta * Elem<OutT>::widen(*p);
                }
                if (fused) x = apply_activation(x + bias, g.act, g.act_param);
                if constexpr (Elem<OutT>::BYTES == 4) *p = as_u32(x);
                else *p = (out_t)Elem<OutT>::narrow(x);
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int col = n0 + wn * WTN + j * 32 + l32;
            const bool col_ok = !EDGE || col < (g.c_cols > 0 ? g.c_cols : g.N);
            if (fused) {                                  // bias and / or activation folded into the store
                const float bias = (g.bias && col_ok) ? g.bias[col] : 0.0f;
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] = apply_activation(acc[i][j][r] + bias, g.act, g.act_param);
            }
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = m0 + wm * WTM + i * 32 + acc_row(r, h);
                out_t* p = C + (long long)row * g.ldc + col;
                out_t v;
                if constexpr (Elem<OutT>::BYTES == 4) v = as_u32(acc[i][j][r]);
                else v = (out_t)Elem<OutT>::narrow(acc[i][j][r]);
                if (col_ok && (!EDGE || row < g.M)) *p = v;
            }
        }
}

template <typename T, typename OutT, bool EDGE = false, int TILE = 256, bool TRANSB = false, int KSW = 1>
static hipError_t launch_gemm_dl(GemmArgs g, int batch, hipStream_t stream)
{
    auto kern = gemm_dl_kernel<T, OutT, EDGE, TILE, TRANSB, KSW>;
    constexpr int smem = 2 * (TILE * 128 + 128 * TILE);         // A tile + B tile (128 bytes of K each), two stages
    static unsigned long long attr_done = 0;
    if (hipError_t e = ensure_dynamic_smem((const void*)kern, smem, &attr_done)) return e;
    g.tiles_m = (g.M + TILE - 1) / TILE;
    g.tiles_n = (g.N + TILE - 1) / TILE;
    hipLaunchKernelGGL(kern, dim3((unsigned)(g.tiles_m * g.tiles_n), 1, (unsigned)batch), dim3((TILE == 256 ? 512 : 256) * KSW), smem, stream, g);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------
// 256 x 256 x 64 direct-to-LDS kernel for 16-bit inputs on v_mfma_f32_16x16x32 (the form the large exact-fit problems take:
// N a multiple of the tile width, K % 64 == 0, B stored [K,N]; M may be ragged: the rows of A past M are clamped loads of row
// M - 1 whose products are never stored).  Same tile, loads and LDS layout as gemm_dl_kernel<.., 256>; what
// differs is the matrix instruction.  Under load this part runs at the clock its power limit allows, and per multiply-add the
// 16 x 16 x 32 instruction moves 20 % fewer register bytes than 32 x 32 x 16 (half the accumulator traffic, twice the
// operand traffic): with random fp16 operands and nothing else running it sustains 1.71 PFLOP/s against 1.52, and this kernel
// 7-10 % more than the 32 x 32 x 16 one on the same box.
//   * wave tile 128 x 64 = 8 x 4 blocks of 16 x 16, 128 accumulator registers; per 32 k: 8 A fragments (ds_read_b128: row
//     16 i + lane % 16, 16-byte chunk lane / 16) and 4 B fragments (two transposing reads each), 32 MFMAs of 16 cycles.
//   * a K-tile is four half-steps of 16 MFMAs (rows 64 hs .. 64 hs + 63 of the wave tile, k32-step s2); the fragments of the
//     next half-step are read one LDS instruction behind each MFMA, the barrier that publishes the next tile sits before the
//     last half-step, whose MFMAs cover the twelve reads of the next tile's first fragments.
//   * the B fragment is the MFMA's first operand, so the accumulators hold C transposed: a lane owns 4 consecutive columns of
//     one row, packs them to 8 bytes, and the wave stages its rows through its 8 KiB of the dead LDS stage so that C leaves as
//     whole 128-byte lines (the 32 x 32 kernel stores 2 bytes per lane and instruction).
//   * MFMA order: one operand changes between consecutive instructions (row-block outer, column-block inner, snaked).
typedef float f32x4_acc __attribute__((ext_vector_type(4)));
template <typename T> struct Mma16;
template <> struct Mma16<f16_t> {
    static __device__ __forceinline__ void run(f32x4_acc& acc, const u32x4& a, const u32x4& b)
    { acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), acc, 0, 0, 0); }
};
template <> struct Mma16<bf16_t> {
    static __device__ __forceinline__ void run(f32x4_acc& acc, const u32x4& a, const u32x4& b)
    { acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0); }
};

// TJ = 16-column blocks per wave: the tile is 256 x (64 TJ) -- 256 x 256, 256 x 192 or 256 x 128 -- so that problems whose 256 x 256
// tiles would leave CUs idle in the last round (4096 x 3072: 192 tiles on 256 CUs) get a tile count that fills them.  The B tile
// keeps its 512-byte LDS rows for every TJ (the chunk swizzle needs a power-of-two row); lanes whose swizzled chunk lies past
// the tile's columns fetch a valid chunk again and park it in a position that no fragment read touches.
// HALF: the 128 x 128 tile (TJ = 2): wave tile 64 x 32, B k-rows of 256 bytes, for problems that give fewer than a chip of wider
// tiles (2048^2, 1024 x 4096).  A K-tile is only 256 MFMA cycles per wave here, far less than a memory round trip, so the tile ring
// has four 32 KB stages and is filled three K-tiles ahead (loads complete in issue order: "tile kt+1 has landed" is a count of
// younger loads).
#define DL16_HALF_STAGES 4
// NTS: C is written with non-temporal stores (a compile-time switch: as a run-time branch the two stores are merged by the compiler
// and the hint is lost).
template <typename T, typename OutT, int TJ = 4, bool HALF = false, bool NTS = false, int HS = DL16_HALF_STAGES>
__global__ __launch_bounds__(512, 1) void gemm_dl16_kernel(const GemmArgs g)
{
    static_assert(!HALF || TJ == 2, "the 128-row tile is built for 128 columns");
    constexpr int E = 8, EB = 2;
    constexpr int WN = 4;
    constexpr int BM = HALF ? 128 : 256, BN = 64 * TJ, BK = 64;
    constexpr int WTM = BM / 2, WTN = 16 * TJ;
    constexpr int TI = WTM / 16;                  // 16 x 16 blocks of the wave tile: TI x TJ
    // LDS pitch of a B k-row (16 or 32 chunk positions): 512 bytes, or 256 for the 128-column tiles (with 512-byte rows the 256 x 128
    // tile fetched 256 columns of B per k-row for the 128 it uses: 6-8 % slower on every shape that takes it)
    constexpr int BROW = ((HALF || TJ == 2) ? 128 : 256) * EB;
    constexpr int BCH = BN / E;                   // 16-byte chunks of a k-row that hold tile columns
    constexpr int ABYTES = BM * 128, BBYTES = BK * BROW, STAGE = ABYTES + BBYTES;
    constexpr int LA = BM / 64, LB = BK * BROW / 8192, RPL = 1024 / BROW, LPR = BROW / 16;
    constexpr int OB = Elem<OutT>::BYTES;

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int l16 = lane & 15, g4 = lane >> 4;
    const int wm = wave / WN, wn = wave % WN;
    int tile_m, tile_n;
    tile_of_block(blockIdx.x, gridDim.x, g.tiles_m, g.tiles_n, tile_m, tile_n);
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const long long bz = blockIdx.z;
    const unsigned char* __restrict__ A = (const unsigned char*)g.A + bz * g.sA * EB;
    const unsigned char* __restrict__ B = (const unsigned char*)g.B + bz * g.sB * EB;

    // Chunk swizzle of a B k-row (position of 16-byte chunk c in its 512-byte LDS row: c ^ b_swz(row)): the four rows one
    // transposing read touches go to different bank groups, and rows 8 apart -- the two 16-lane groups that share a cycle of
    // that read -- are moved 32 bytes apart.
    auto b_swz = [](int row) -> int { return ((row & 3) << 2) | (((row >> 3) & 1) << 1); };
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)smem);
    // A rows past M (the last tile row of a ragged M) are clamped to row M - 1: valid loads whose products are never stored
    uint32_t a_lane_off[LA], b_lane_off[LB];
#pragma unroll
    for (int i = 0; i < LA; i++) {
        const int ra = lane >> 3, pos_a = lane & 7;
        const int row = min(m0 + 8 * (LA * wave + i) + ra, g.M - 1) - m0;        // relative to the tile's first row, >= 0
        a_lane_off[i] = (uint32_t)(row * g.lda + (pos_a ^ ((4 * (i & 1) + (ra >> 1)) & 7)) * E) * (uint32_t)EB;
    }
#pragma unroll
    for (int i = 0; i < LB; i++) {
        const int rb = lane / LPR, pos_b = lane % LPR;
        int chunk = pos_b ^ b_swz(RPL * (LB * wave + i) + rb);
        if (chunk >= BCH) chunk -= LPR - BCH >= BCH ? BCH : LPR - BCH;    // a valid chunk again (its LDS position is never read)
        b_lane_off[i] = (uint32_t)(rb * g.ldb + chunk * E) * (uint32_t)EB;
    }
    const unsigned char* a_base = A + (long long)m0 * g.lda * EB;
    const unsigned char* b_base = B + ((long long)(RPL * LB * wave_s) * g.ldb + n0) * EB;
    const long long b_step = (long long)RPL * g.ldb * EB;
    const int KT = g.K / BK;
    auto issue_loads = [&](int kt, int stage) {
        const uint32_t as = lds0 + stage * STAGE + wave_s * (LA * 1024);
        const uint32_t bs = lds0 + stage * STAGE + ABYTES + wave_s * (LB * 1024);
        const unsigned char* a_src = a_base + (long long)kt * 128;
        const unsigned char* b_src = b_base + (long long)kt * BK * g.ldb * EB;
#pragma unroll
        for (int i = 0; i < LA; i++) dma16_base(a_src, a_lane_off[i], as + i * 1024);
#pragma unroll
        for (int i = 0; i < LB; i++) dma16_base(b_src + i * b_step, b_lane_off[i], bs + i * 1024);
    };

    // A fragment of 16-row block i, k32-step s2: row 16 i + l16, chunk 4 s2 + g4, swizzled by (row >> 1) & 7 = (l16 >> 1) & 7
    const int a_row0 = (wm * WTM + l16) * 128;
    const int a_sw = (l16 >> 1) & 7;
    // B fragment of 16-column block j, k32-step s2: two transposing reads (q = 0, 1); the lane addresses k-row
    // 32 s2 + 8 g4 + 4 q + l16 / 4 and the 8 bytes at column 16 j + 4 (l16 % 4), and receives k 8 g4 + 4 q .. + 3 of column 16 j + l16
    const int b_rowl = 8 * g4 + (l16 >> 2);
    const int b_half = (l16 & 1) * 8;
    const int b_chunk0 = wn * (2 * TJ) + ((l16 & 3) >> 1);      // + 2 j

    auto read_a = [&](const unsigned char* as, int s2, int i, u32x4& f) {
        f = *(const u32x4*)(as + a_row0 + i * 2048 + (((4 * s2 + g4) ^ a_sw) << 4));
    };
    auto read_b = [&](const unsigned char* bs, int s2, int j, u32x4& f) {
#pragma unroll
        for (int q = 0; q < 2; q++) {
            const int row = 32 * s2 + 4 * q + b_rowl;
            const int pos = (b_chunk0 + 2 * j) ^ b_swz(row);
            s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                (__attribute__((address_space(3))) s16x4*)(bs + row * BROW + pos * 16 + b_half));
            u32x2 w = __builtin_bit_cast(u32x2, v);
            f[2 * q] = w[0];
            f[2 * q + 1] = w[1];
        }
    };

    f32x4_acc acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < TJ; j++) acc[i][j] = f32x4_acc{0.0f, 0.0f, 0.0f, 0.0f};

    constexpr int NS = HALF ? HS : 2;
    // wait until at most `tiles` of this wave's tile loads (LA + LB instructions each) are outstanding, and for its LDS reads
    auto wait_tiles = [&](int tiles) {
        static_assert(!HALF || (LA + LB == 4 && NS <= 4), "the wait counts below are for four loads per tile and a four-stage ring");
        if (tiles <= 0) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        else if (tiles == 1) asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory");
    };
    if constexpr (HALF) {
        for (int kt = 0; kt < NS - 1 && kt < KT; kt++) issue_loads(kt, kt);
        wait_tiles(min(KT - 1, NS - 2));
    } else {
        issue_loads(0, 0);
        __builtin_amdgcn_s_waitcnt(0);
    }
    __syncthreads();

    // fa[p]: the four A fragments of half-step parity p; fb[p]: the four B fragments of k32-step parity p
    u32x4 fa[2][4], fb[2][TJ];
#pragma unroll
    for (int i = 0; i < 4; i++) read_a(smem, 0, i, fa[0][i]);
#pragma unroll
    for (int j = 0; j < TJ; j++) read_b(smem + ABYTES, 0, j, fb[0][j]);

    if constexpr (HALF) {
        // two steps per K-tile (one k32-step each, the whole 64-row wave tile): 8 MFMAs and 8 LDS reads per step
        int stage = 0;
        for (int kt = 0; kt < KT; kt++) {
            const int next = stage + 1 == NS ? 0 : stage + 1;
            const unsigned char* as = smem + stage * STAGE;
            const unsigned char* bs = as + ABYTES;
            const unsigned char* an = smem + next * STAGE;
            // the stage of tile kt-1 was last read before the barrier inside the previous iteration
            if (kt + NS - 1 < KT) issue_loads(kt + NS - 1, stage == 0 ? NS - 1 : stage - 1);
#pragma unroll
            for (int s2 = 0; s2 < 2; s2++) {
                if (s2 == 0) {
#pragma unroll
                    for (int i = 0; i < 4; i++) read_a(as, 1, i, fa[1][i]);
#pragma unroll
                    for (int j = 0; j < TJ; j++) read_b(bs, 1, j, fb[1][j]);
                } else {
                    wait_tiles(min(KT - 2 - kt, NS - 2));   // this wave's part of tile kt+1 has landed (younger tiles may be in flight), its LDS reads of tile kt are done ...
                    __syncthreads();                        // ... and so have everyone else's
                    if (kt + 1 < KT) {
#pragma unroll
                        for (int i = 0; i < 4; i++) read_a(an, 0, i, fa[0][i]);
#pragma unroll
                        for (int j = 0; j < TJ; j++) read_b(an + ABYTES, 0, j, fb[0][j]);
                    }
                }
#pragma unroll
                for (int i = 0; i < 4; i++)
#pragma unroll
                    for (int jj = 0; jj < TJ; jj++) {
                        const int j = (i & 1) ? TJ - 1 - jj : jj;
                        Mma16<T>::run(acc[i][j], fb[s2][j], fa[s2][i]);
                    }
                constexpr int NM = 4 * TJ, RR = 4 + 2 * TJ;
                spread_schedule<RR, RR, 0, 0>();
                if (NM > RR) __builtin_amdgcn_sched_group_barrier(0x008, NM - RR, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
            stage = next;
        }
    } else {
    for (int kt = 0; kt < KT; kt++) {
            const int stage = kt & 1;
            const unsigned char* as = smem + stage * STAGE;
            const unsigned char* bs = as + ABYTES;
            const unsigned char* an = smem + (stage ^ 1) * STAGE;
            // the other stage was last read before the barrier inside the previous iteration
            if (kt + 1 < KT) issue_loads(kt + 1, stage ^ 1);
    #pragma unroll
            for (int u = 0; u < 4; u++) {              // half-step u = 2 s2 + hs
                const int s2 = u >> 1, hs = u & 1;
                if (u == 0) {
    #pragma unroll
                    for (int i = 0; i < 4; i++) read_a(as, 0, 4 + i, fa[1][i]);
                    read_b(bs, 1, 0, fb[1][0]); read_b(bs, 1, 1, fb[1][1]);
                } else if (u == 1) {
    #pragma unroll
                    for (int i = 0; i < 4; i++) read_a(as, 1, i, fa[0][i]);
    #pragma unroll
                    for (int j = 2; j < TJ; j++) read_b(bs, 1, j, fb[1][j]);
                } else if (u == 2) {
    #pragma unroll
                    for (int i = 0; i < 4; i++) read_a(as, 1, 4 + i, fa[1][i]);
                } else {
                    __builtin_amdgcn_s_waitcnt(0);      // this wave's DMA has landed and its LDS reads of this tile are done ...
                    __syncthreads();                    // ... and so have everyone else's
                    if (kt + 1 < KT) {
    #pragma unroll
                        for (int i = 0; i < 4; i++) read_a(an, 0, i, fa[0][i]);
    #pragma unroll
                        for (int j = 0; j < TJ; j++) read_b(an + ABYTES, 0, j, fb[0][j]);
                    }
                }
    #pragma unroll
                for (int i = 0; i < 4; i++)
    #pragma unroll
                    for (int jj = 0; jj < TJ; jj++) {
                        const int j = (i & 1) ? TJ - 1 - jj : jj;
                        Mma16<T>::run(acc[4 * hs + i][j], fb[s2][j], fa[hs][i]);
                    }
                // one LDS read behind each of the first MFMAs, the remaining MFMAs after the reads have been issued
                constexpr int NM = 4 * TJ;                                   // MFMAs per half-step
                constexpr int R0 = 8, R1 = 4 + 2 * (TJ - 2), R2 = 4, R3 = 4 + 2 * TJ;      // LDS reads of the four half-steps
                if (u == 0) { spread_schedule<R0, R0, 0, 0>(); __builtin_amdgcn_sched_group_barrier(0x008, NM - R0, 0); }
                else if (u == 1) { spread_schedule<R1, R1, 0, 0>(); __builtin_amdgcn_sched_group_barrier(0x008, NM - R1, 0); }
                else if (u == 2) { spread_schedule<R2, R2, 0, 0>(); __builtin_amdgcn_sched_group_barrier(0x008, NM - R2, 0); }
                else { spread_schedule<R3, R3, 0, 0>(); __builtin_amdgcn_sched_group_barrier(0x008, NM - R3, 0); }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    
}

    // ---- epilogue.  acc[i][j]: the lane holds C[row 16 i + l16][columns 16 j + 4 g4 .. + 3].  Staged through the wave's 8 KiB of
    // the last stage (dead after the final barrier), 16-byte chunk c of a staged row at position c ^ ((row >> 1) & 7).
    {
        // (HALF: every stage is dead after the final barrier; the eight waves' 8 KiB take the first two)
        // (the eight waves' 64 KiB may reach past a 48 KiB stage into the other one, which is just as dead; the launch allocates 128 KiB)
        static_assert(HALF || STAGE + 8 * 8192 <= 2 * (256 * 128 + 128 * 256), "C staging must stay inside the allocation");
        unsigned char* stg = smem + (HALF ? 0 : ((KT - 1) & 1) * STAGE) + wave * 8192;
        constexpr int ROWB = WTN * OB;                // bytes of one staged row
        constexpr int CPR = ROWB / 16;                // 16-byte chunks per staged row
        constexpr bool POW2 = (CPR & (CPR - 1)) == 0; // the XOR swizzle of the staged rows needs a power-of-two chunk count
        // (rows of another width, the 96 columns a wave holds of a 192-wide tile, are staged 16 bytes apart from whole rows instead: the
        // pad moves neighbouring rows onto different banks, where unpadded rows cost a fifth of the LDS cycles of that tile in conflicts)
        constexpr int PITCH = POW2 ? ROWB : ROWB + 16;
        constexpr int FIT = 8192 / (16 * PITCH);      // 16-row blocks that fit the wave's 8 KiB
        constexpr int IPR0 = FIT >= 8 ? 8 : FIT >= 4 ? 4 : FIT >= 2 ? 2 : 1;
        constexpr int IPR = IPR0 < TI ? IPR0 : TI;    // blocks per round (divides TI)
        const int sw = POW2 ? ((l16 >> 1) & (CPR - 1) & 7) : 0;
        const bool fused = g.bias != nullptr || g.act != 0;
        f32x4 bias4[TJ];
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            bias4[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            if (g.bias) bias4[j] = *(const f32x4*)(g.bias + n0 + wn * WTN + 16 * j + 4 * g4);
        }
        unsigned char* Cw = (unsigned char*)g.C + (bz * g.sC + (long long)(m0 + wm * WTM) * g.ldc + n0 + wn * WTN) * OB;
        const bool whole_tile = __builtin_amdgcn_readfirstlane(m0 + (HALF ? 128 : 256) <= g.M && g.c_cols == 0);
        static_for<0, TI, IPR>([&](auto ip_const) {
            constexpr int ip = decltype(ip_const)::value;
#pragma unroll
            for (int ii = 0; ii < IPR; ii++) {
#pragma unroll
                for (int j = 0; j < TJ; j++) {
                    f32x4_acc v = acc[ip + ii][j];
                    if (fused) {
#pragma unroll
                        for (int e = 0; e < 4; e++) v[e] = apply_activation(v[e] + bias4[j][e], g.act, g.act_param);
                    }
                    const int row = ii * 16 + l16;
                    if constexpr (OB == 2) {
                        const uint32_t w0 = Elem<OutT>::narrow(v[0]) | (Elem<OutT>::narrow(v[1]) << 16);
                        const uint32_t w1 = Elem<OutT>::narrow(v[2]) | (Elem<OutT>::narrow(v[3]) << 16);
                        const int chunk = 2 * j + (g4 >> 1);
                        *(u32x2*)(stg + row * PITCH + ((chunk ^ sw) << 4) + (g4 & 1) * 8) = u32x2{w0, w1};
                    } else {
                        const int chunk = 4 * j + g4;
                        *(u32x4*)(stg + row * PITCH + ((chunk ^ sw) << 4)) = u32x4{as_u32(v[0]), as_u32(v[1]), as_u32(v[2]), as_u32(v[3])};
                    }
                }
            }
            // a workgroup whose tile lies inside the matrix (every one but the last tile row of a ragged M) stores without a
            // test per row: with the test the compiler serialises LDS read and store of every chunk, which costs the short-K
            // shapes 3-5 %
            if (whole_tile) {
#pragma unroll
                for (int q = 0; q < IPR * 16 * CPR / 64; q++) {
                    const int u = q * 64 + lane;
                    const int row = u / CPR, c = u % CPR;
                    const u32x4 v = *(const u32x4*)(stg + row * PITCH + ((c ^ (POW2 ? ((row >> 1) & (CPR - 1) & 7) : 0)) << 4));
                    u32x4* dst = (u32x4*)(Cw + (long long)(ip * 16 + row) * g.ldc * OB + c * 16);
                    if constexpr (NTS) __builtin_nontemporal_store(v, dst);
                    else *dst = v;
                }
            } else {
                // (a rolled loop: nothing in it is indexed by q at compile time, and unrolled it grows the epilogue so much that
                // the compiler stops unrolling the loop over ip, whose accumulator indices must be constants)
#pragma unroll 1
                for (int q = 0; q < IPR * 16 * CPR / 64; q++) {
                    const int u = q * 64 + lane;
                    const int row = u / CPR, c = u % CPR;
                    const u32x4 v = *(const u32x4*)(stg + row * PITCH + ((c ^ (POW2 ? ((row >> 1) & (CPR - 1) & 7) : 0)) << 4));
                    u32x4* dst = (u32x4*)(Cw + (long long)(ip * 16 + row) * g.ldc * OB + c * 16);
                    if (m0 + wm * WTM + ip * 16 + row >= g.M) continue;
                    if (g.c_cols > 0) {
                        // rows of C at any element offset: whole chunks by one under-aligned 16-byte store, the chunk that
                        // crosses the last column by elements
                        typedef typename Raw<OutT>::type out_t;
                        typedef u32x4 u32x4_elem __attribute__((aligned(2)));
                        constexpr int PER = 16 / OB;
                        const int col0 = n0 + wn * WTN + c * PER;
                        if (col0 + PER <= g.c_cols) *(u32x4_elem*)dst = v;
                        else {
#pragma unroll
                            for (int e = 0; e < PER; e++)
                                if (col0 + e < g.c_cols) {
                                    if constexpr (OB == 2) ((out_t*)dst)[e] = (out_t)(v[e >> 1] >> ((e & 1) * 16));
                                    else ((out_t*)dst)[e] = v[e];
                                }
                        }
                    } else *dst = v;
                }
            }
        });
    }
}

template <typename T, typename OutT, int TJ = 4, bool HALF = false, int HS = DL16_HALF_STAGES>
static hipError_t launch_gemm_dl16(GemmArgs g, int batch, hipStream_t stream)
{
    constexpr int smem = HALF ? HS * (128 * 128 + 64 * 256) : 2 * (256 * 128 + 128 * 256);
    g.tiles_m = (g.M + (HALF ? 127 : 255)) / (HALF ? 128 : 256);      // the last tile row may be partial
    g.tiles_n = g.N / (64 * TJ);
    const dim3 grid((unsigned)(g.tiles_m * g.tiles_n), 1, (unsigned)batch);
    // Non-temporal stores of C when A, B and C together exceed the 256 MB last-level cache: C then no longer displaces the operand
    // tiles that later workgroups re-read (alternated in one process: fp16 8192^3 1336 -> 1408 TFLOP/s, bf16 1397 -> 1464,
    // 16384 x 8192 x 1024 989 -> 1166, 8192 x 50304 x 768 764 -> 873); a problem that fits the cache is better left to its
    // write-back path (4096 x 3072 x 768 881 -> 770, 8192 x 8192 x 2048 1283 -> 1248 with such stores).
    const long long footprint = ((long long)g.M * g.K + (long long)g.K * g.N) * 2 * batch + (long long)g.M * g.N * batch * Elem<OutT>::BYTES;
    const bool nts = footprint > (240LL << 20);
    if constexpr (!HALF) {
        if (nts) {
            auto kern = gemm_dl16_kernel<T, OutT, TJ, false, true>;
            static unsigned long long attr_done_nt = 0;
            if (hipError_t e = ensure_dynamic_smem((const void*)kern, smem, &attr_done_nt)) return e;
            hipLaunchKernelGGL(kern, grid, dim3(512), smem, stream, g);
            return hipGetLastError();
        }
    }
    auto kern = gemm_dl16_kernel<T, OutT, TJ, HALF, false, HS>;
    static unsigned long long attr_done = 0;
    if (hipError_t e = ensure_dynamic_smem((const void*)kern, smem, &attr_done)) return e;
    hipLaunchKernelGGL(kern, grid, dim3(512), smem, stream, g);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------
// Skinny-M path (decode projections): M <= 32, 16-bit, B stored [K,N], N % 128 == 0, K % 64 == 0.
// HBM-bound: B (K x N) is read exactly once.  grid = (N / 128, KS), about one workgroup per CU: each workgroup streams a
// 128-column slab of B over its K range with the direct global->LDS load through a ring of NS 20 KB stages, filled NS - 1
// K-tiles ahead -- seven stages and one workgroup per CU (120 KB in flight per CU: one memory round trip covers a whole K range of
// up to six tiles, where a two-stage ring paid one round trip per tile), or three stages and two workgroups per CU for wide
// weights (launch_skinny) --, computes a 32 x 128 partial product on MFMA (A rows beyond M are
// clamped duplicates that are never stored) and writes it to an fp32 workspace that skinny_reduce_kernel sums in split order
// (deterministic) and narrows.  Loads complete in issue order, so "tile kt has landed" is a count of younger loads.
//   B tile [64 k][256 B]: chunk c of row k at position c ^ ((k & 3) << 2)   (transposing reads)
//   A tile [32 m][128 B]: chunk c of row m at position c ^ ((m >> 1) & 7)   (b128 reads)
#define SKINNY_STAGES 7
template <typename T, int NS>
__global__ __launch_bounds__(256, NS <= 3 ? 2 : 1) void gemm_skinny_kernel(const GemmArgs g, float* __restrict__ ws, int ksplit, int kper)
{
    typedef uint16_t raw_t;
    constexpr int BK = 64, AHEAD = NS - 1;
    constexpr int ABYTES = 32 * 128, BBYTES = BK * 256, STAGE = ABYTES + BBYTES;
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];      // NS stages

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    const int n0 = blockIdx.x * 128;
    const int ks = blockIdx.y;
    const int kbeg = ks * kper;
    const int KT = min(kper, g.K - kbeg) / BK;            // the last range may be shorter
    const raw_t* __restrict__ A = (const raw_t*)g.A;
    const raw_t* __restrict__ B = (const raw_t*)g.B;

    // this wave's DMA per K-tile: 4 B wave-loads (k-rows 4w'..4w'+3, w' = 4*wave+i) and A wave-load `wave` (rows 8*wave..)
    const raw_t* pb[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        int row = 4 * (wave * 4 + i) + (lane >> 4), pos = lane & 15;
        pb[i] = B + (long long)(kbeg + row) * g.ldb + n0 + (pos ^ ((row & 3) << 2)) * 8;
    }
    const raw_t* pa;
    {
        int row = 8 * wave + (lane >> 3), pos = lane & 7;
        int grow = min(row, g.M - 1);
        pa = A + (long long)grow * g.lda + kbeg + (pos ^ ((row >> 1) & 7)) * 8;
    }
    auto issue_loads = [&](int kt, int stage) {
        unsigned char* as = smem + stage * STAGE;
        unsigned char* bs = as + ABYTES;
        dma16_to_lds(pa + kt * BK, as + wave * 1024);
#pragma unroll
        for (int i = 0; i < 4; i++) dma16_to_lds_stream(pb[i] + (long long)kt * BK * g.ldb, bs + (wave * 4 + i) * 1024);
    };

    const int a_off = l32 * 128, a_sw = (l32 >> 1) & 7;
    const int jl = lane & 15;
    const int b_rowl = 8 * h + (jl >> 2);
    const int b_half = (jl & 1) * 8;
    const int b_chunk = (wave * 32 + 16 * ((lane >> 4) & 1) + 4 * (jl & 3)) >> 3;

    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.0f;

    for (int kt = 0; kt < AHEAD && kt < KT; kt++) issue_loads(kt, kt);
    int stage = 0;
    for (int kt = 0; kt < KT; kt++) {
        // tiles kt+1 .. kt+AHEAD-1 (those that exist) are younger than tile kt: five loads per wave each
        switch (min(KT - 1 - kt, AHEAD - 1)) {
            case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
            case 1: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
            case 2: asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); break;
            case 3: asm volatile("s_waitcnt vmcnt(15)" ::: "memory"); break;
            case 4: asm volatile("s_waitcnt vmcnt(20)" ::: "memory"); break;
            default: asm volatile("s_waitcnt vmcnt(25)" ::: "memory"); break;
        }
        __syncthreads();            // everyone's part of tile kt has landed, and everyone has left tile kt-1
        if (kt + AHEAD < KT) issue_loads(kt + AHEAD, stage == 0 ? NS - 1 : stage - 1);      // into the stage tile kt-1 used
        const unsigned char* as = smem + stage * STAGE;
        const unsigned char* bs = as + ABYTES;
#pragma unroll
        for (int s = 0; s < 4; s++) {
            u32x4 fa = *(const u32x4*)(as + a_off + (((2 * s + h) ^ a_sw) << 4));
            u32x4 fb;
#pragma unroll
            for (int q = 0; q < 2; q++) {
                int row = 16 * s + 4 * q + b_rowl;
                int pos = b_chunk ^ ((row & 3) << 2);
                s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (__attribute__((address_space(3))) s16x4*)(bs + row * 256 + pos * 16 + b_half));
                u32x2 w = __builtin_bit_cast(u32x2, v);
                fb[2 * q] = w[0];
                fb[2 * q + 1] = w[1];
            }
            Mma32<T>::run(acc, fa, fb);
        }
        stage = stage + 1 == NS ? 0 : stage + 1;
    }

    const int col = n0 + wave * 32 + l32;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int row = acc_row(r, h);
        if (row < g.M) ws[((long long)ks * g.M + row) * g.N + col] = acc[r];
    }
}

template <typename OutT>
__global__ __launch_bounds__(256) void skinny_reduce_kernel(const float* __restrict__ ws, void* __restrict__ Cv, int M, int N, int ksplit,
                                                             const float* __restrict__ bias, int act, float act_param,
                                                             float alpha = 1.0f, float beta = 0.0f)
{
    typedef typename Raw<OutT>::type out_t;
    out_t* C = (out_t*)Cv;
    const long long total = (long long)M * N;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
        float s = 0.0f;
        int k = 0;
        for (; k + 8 <= ksplit; k += 8) {              // eight loads in flight, summed in split order
            float t[8];
#pragma unroll
            for (int u = 0; u < 8; u++) t[u] = ws[(long long)(k + u) * total + i];
#pragma unroll
            for (int u = 0; u < 8; u++) s += t[u];
        }
        for (; k < ksplit; k++) s += ws[(long long)k * total + i];
        if constexpr (Elem<OutT>::BYTES == 4) {
            s *= alpha;
            if (beta != 0.0f) s += beta * as_f32(C[i]);
        }
        if (bias) s += bias[i % N];
        s = apply_activation(s, act, act_param);
        if constexpr (Elem<OutT>::BYTES == 4) C[i] = as_u32(s);
        else C[i] = (out_t)Elem<OutT>::narrow(s);
    }
}

// The summing pass with the rotary embedding on top: one thread per column pair (2 j, 2 j + 1) of a row sums both columns in split
// order, rotates the pair when it lies in the first rope.cols columns, and stores both with one rounding.
template <typename OutT>
__global__ __launch_bounds__(256) void skinny_reduce_rope_kernel(const float* __restrict__ ws, uint16_t* __restrict__ C, int M, int N, int ksplit,
                                                                  const RopeEpilogue rope)
{
    typedef float f32x2a __attribute__((ext_vector_type(2)));
    const long long total = (long long)M * N, pairs = total >> 1;
    const int half = rope.head_dim >> 1, row_pairs = N >> 1;
    for (long long p = (long long)blockIdx.x * blockDim.x + threadIdx.x; p < pairs; p += (long long)gridDim.x * blockDim.x) {
        float s0 = 0.0f, s1 = 0.0f;
        for (int k = 0; k < ksplit; k++) {
            const f32x2a t = *(const f32x2a*)(ws + (long long)k * total + 2 * p);
            s0 += t[0]; s1 += t[1];
        }
        const int m = (int)(p / row_pairs), col = 2 * (int)(p - (long long)m * row_pairs);
        if (col < rope.cols) {
            const int i = (col % rope.head_dim) >> 1;
            const long long pos = rope.start_position + m % rope.seq_len;
            // (the pair is rounded to the output type before it is rotated: what a product followed by the rotation kernel computes)
            const float xe = Elem<OutT>::widen(Elem<OutT>::narrow(s0)), xo = Elem<OutT>::widen(Elem<OutT>::narrow(s1));
            rope_rotate(xe, xo, rope.cosc[pos * half + i], rope.sinc[pos * half + i], s0, s1);
        }
        ((uint32_t*)C)[p] = Elem<OutT>::narrow(s0) | (Elem<OutT>::narrow(s1) << 16);
    }
}

static bool skinny_applies(int M, int N, int K) { return M <= 32 && N % 128 == 0 && K % 64 == 0 && N >= 128; }

// How evenly `tiles` workgroups load the 256 CUs: a CU works through its tiles at about the same rate whether it holds one or
// several at a time, so what counts is the largest number of tiles any CU gets.
static double cu_fill(long long tiles) { return (double)tiles / (double)(((tiles + 255) / 256) * 256); }

// K ranges of the skinny paths: `tiles` K-tiles over `slabs` column slabs, one workgroup per CU at a time.  Returns the K-tiles per
// range (the last range may be shorter); *ks = number of ranges.  Scored as (how evenly slabs x ranges load the 256 CUs) x (the
// share of a workgroup's time that is not its first memory round trip, about three K-tiles' worth).
static int skinny_plan(int slabs, int tiles, int* ks_out, int per_cu = 1, double* score_out = nullptr)
{
    int best_kper = tiles, best_ks = 1;
    double best = -1.0;
    const long long slots = 256LL * per_cu;
    // (two workgroups per CU: one's first round trip runs under the other's stream, so it counts half)
    const double ramp = per_cu == 1 ? 3.0 : 1.5;
    for (int ks = 1; ks <= 32 && ks <= tiles; ks++) {
        const int kper = (tiles + ks - 1) / ks;
        const int kse = (tiles + kper - 1) / kper;
        if (kper < 4 && ks > 1) break;
        const long long wg = (long long)slabs * kse;
        const double fill = (double)wg / (double)(((wg + slots - 1) / slots) * slots);
        const double score = fill * (double)kper / (kper + ramp);
        if (score > best * 1.02) { best = score; best_kper = kper; best_ks = kse; }
    }
    *ks_out = best_ks;
    if (score_out) *score_out = best;
    return best_kper;
}
static int skinny_ksplit(int N, int K) { int ks; skinny_plan(N / 128, K / 64, &ks, N / 128 > 64 && K <= 4096 ? 2 : 1); return ks; }

// Split-K for 16-bit problems whose 128 x 128 tiles fill less than half the chip over a long K (M <= 512 against a 4096-wide
// weight): K ranges run as the batch dimension of the 128 x 128 kernel into fp32 partials, summed in range order by
// skinny_reduce_kernel (deterministic; bias and activation there).  Returns the number of ranges, 0 = not worth it.
static int dl16_width(int M, int N, int K, int batch, double* score_out = nullptr);
// Share of a split-K product's time that is the product: the fp32 partials are written and read once per range, 8 bytes per output
// element and range at about 4 TB/s, against 2 K flops per element at about 1.4 PFLOP/s (512 x 8192 x 8192 in four ranges: 49 us of
// product, 33 us of partials)
static double splitk16_partials_factor(int K, int ks) { return 1.0 / (1.0 + 1000.0 * ks / K); }
static int splitk16_ranges(int M, int N, int K, int* big_tile = nullptr)
{
    if (big_tile) *big_tile = 0;
    if (N % 128 != 0 || K % 64 != 0) return 0;
    auto ranges = [&](long long t, int min_k) {
        int ks = (int)(256 / t);
        if (ks > 16) ks = 16;
        while (ks > 1 && (K % (ks * 64) != 0 || K / ks < min_k)) ks--;
        return ks;
    };
    // (a ragged M: the last tile row is partial)
    const long long t = (long long)((M + 127) / 128) * (N / 128);
    if (t <= 128) {                           // up to half a chip of 128 x 128 tiles
        const int ks = ranges(t, 512);
        // the partials cost 8 bytes of traffic per output element and range; the product must be worth it
        // (a ragged M only from K = 2048 on: below, the second launch costs what the ranges save -- 1000 x 1024 x 1024 8 -> 15 us)
        return ks >= 2 && (long long)K >= (M % 128 == 0 ? 1024 : 2048) ? ks : 0;
    }
    // Larger problems whose 256 x 256 tiles still fill at most half the chip over a long K (M about 1000 against an 8192-wide
    // weight with K = 28672): narrower tiles would fill the chip but move twice the operand bytes per flop through the L2, which
    // is what bounds them at this K; K ranges of the 256 x 256 tile keep its traffic.
    if (N % 256 != 0) return 0;
    const long long t256 = (long long)((M + 255) / 256) * (N / 256);
    if (t256 > 128 || K < 4096) return 0;
    const int ks = ranges(t256, 2048);
    if (ks < 2 || !big_tile) return 0;
    // against the best single launch, by the scores of the tile choice (CU fill x rate per flop x share of real rows)
    double single = 0.0;
    dl16_width(M, N, K, 1, &single);
    const double split = cu_fill(t256 * ks) * ((double)M / (double)(((M + 255) / 256) * 256)) * splitk16_partials_factor(K, ks);
    if (split <= 1.05 * single) return 0;
    *big_tile = 1;
    return ks;
}

// Rows of a tall 16-bit problem to run as a launch of their own: with N / 256 tile columns that divide the 256 CUs, whole rounds of
// 256 x 256 tiles cover a multiple of 256 * 256 / (N / 256) rows at the full rate; the rows that would start a partly filled round
// (3000 rows against an 8192-wide weight: 1.5 rounds) are better served by whatever suits them alone -- narrower tiles, or K
// ranges of the 256 x 256 tile.  Returns the row count of the first launch, 0 = one launch.  Both estimates are rows / score.
static int msplit16_rows(int M, int N, int K)
{
    if (N % 256 != 0 || K % 64 != 0 || 256 % (N / 256) != 0) return 0;
    const int rows_per_round = 256 / (N / 256) * 256;
    const int first = M / rows_per_round * rows_per_round;
    const int rest = M - first;
    if (first == 0 || rest == 0) return 0;
    auto score = [&](int m) {
        double single = 0.0;
        dl16_width(m, N, K, 1, &single);
        int big = 0;
        const int ks = splitk16_ranges(m, N, K, &big);
        if (ks && big) {
            const long long t256 = (long long)((m + 255) / 256) * (N / 256);
            const double split = cu_fill(t256 * ks) * ((double)m / (double)(((m + 255) / 256) * 256)) * splitk16_partials_factor(K, ks);
            if (split > single) single = split;
        }
        return single;
    };
    const double whole = score(M), tail = score(rest);
    if (whole <= 0.0 || tail <= 0.0) return 0;
    return (double)first + (double)rest / tail < 0.92 * (double)M / whole ? first : 0;
}

// 16-bit problems whose rows are not 16-byte aligned (N or K not a multiple of 8) would run on 2-byte loads, an order of
// magnitude below the vector-load kernels.  They are copied instead into zero-padded, aligned operands in the workspace
// (K up to a multiple of 64, N up to a multiple of 128, or of 8 for a narrow N), multiplied there by the kernels for aligned
// problems and the columns of C copied back: three extra passes over A, B and C, which a product of this size repays many
// times over.  The zero columns of A meet zero rows of B, so the padded product holds exactly the sums of the plain one.
struct PadPlan {
    int Np, Kp;                                   // padded N and K
    size_t a_off, b_off, c_off, bias_off, inner_off, total;
};
static size_t gemm_16_inner_workspace_bytes(int M, int N, int K)
{
    size_t need = 0;
    if (skinny_applies(M, N, K)) need = (size_t)skinny_ksplit(N, K) * M * N * sizeof(float);
    if (const int first = msplit16_rows(M, N, K)) {
        const size_t a = gemm_16_inner_workspace_bytes(first, N, K), b = gemm_16_inner_workspace_bytes(M - first, N, K);
        if (a > need) need = a;
        if (b > need) need = b;
    }
    int big;
    const int ks = splitk16_ranges(M, N, K, &big);
    const size_t split = ks ? (size_t)ks * M * N * sizeof(float) : 0;
    return split > need ? split : need;
}
// the padded shapes and the workspace layout for them (no judgement on whether padding pays)
static bool pad16_layout(int M, int N, int K, PadPlan* pl)
{
    const int Np = N >= 512 ? (N + 127) / 128 * 128 : (N + 7) / 8 * 8;
    const int Kp = (K + 63) / 64 * 64;
    auto up = [](size_t b) { return (b + 255) & ~(size_t)255; };
    size_t off = 0;
    pl->Np = Np; pl->Kp = Kp;
    pl->a_off = off; off += up((size_t)M * Kp * 2);
    pl->b_off = off; off += up((size_t)Kp * Np * 2);
    pl->c_off = off; off += up((size_t)M * Np * 4);
    pl->bias_off = off; off += up((size_t)Np * 4);
    pl->inner_off = off; off += gemm_16_inner_workspace_bytes(M, Np, Kp);
    pl->total = off;
    return off <= ((size_t)4 << 30);
}
static bool pad16_plan(int M, int N, int K, PadPlan* pl)
{
    if (N % 8 == 0 && K % 8 == 0) return false;
    if (N < 16 || (double)M * N * K < (double)(1 << 21)) return false;        // launch-bound either way
    // few rows over a short K: the copy of B would cost more than the product; the general kernel reads such rows in place with
    // element-aligned 16-byte loads (64 x 50257 x 768: 42 us against 51 us through the copies)
    if (M <= 512 && K <= 1024) return false;
    return pad16_layout(M, N, K, pl);
}

// dst [rows_dst, cols_dst] (16-byte aligned rows) <- src [rows_src, cols_src] (dense, any alignment), zeros elsewhere; E = element.
// One thread fills one 16-byte chunk of dst from element loads.
template <typename E>
__global__ __launch_bounds__(256) void pad_rows_kernel(const E* __restrict__ src, E* __restrict__ dst, int rows_src, int cols_src,
                                                       int rows_dst, int cols_dst)
{
    constexpr int PER = 16 / (int)sizeof(E);
    typedef E Vec __attribute__((ext_vector_type(PER)));
    const int per_row = cols_dst / PER;
    const long long total = (long long)rows_dst * per_row;
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long g = (long long)blockIdx.x * blockDim.x + threadIdx.x; g < total; g += stride) {
        const long long row = g / per_row;
        const int c0 = (int)(g - row * per_row) * PER;
        Vec v;
#pragma unroll
        for (int e = 0; e < PER; e++) v[e] = (row < rows_src && c0 + e < cols_src) ? src[row * cols_src + c0 + e] : (E)0;
        *(Vec*)(dst + row * cols_dst + c0) = v;
    }
}

// The same for 2-byte elements with every access a dword that is contiguous across the wave: one thread per dword of dst
// (columns 2 i, 2 i + 1 of a row).  A source row starts on a dword boundary or 2 bytes past one; in the second case the two
// elements come from the high half of one source dword and the low half of the next.  A dword of the source is only loaded whole
// when both of its elements belong to the array.  grid = (ceil(cols_dst / 512), rows): no division per thread.
#if AIDN_GEMM_PART == 0
__global__ __launch_bounds__(256) void pad_rows16_kernel(const uint16_t* __restrict__ src, uint32_t* __restrict__ dst, int rows_src, int cols_src,
                                                         int rows_dst, int cols_dst)
{
    const int i = blockIdx.x * 256 + threadIdx.x;                    // dword column of dst
    const int per_row = cols_dst >> 1;
    if (i >= per_row) return;
    const uint32_t* base = (const uint32_t*)(((uintptr_t)src) & ~(uintptr_t)3);
    const long long off0 = (((uintptr_t)src) & 2) ? 1 : 0;           // flat element index of src[0] counted from base
    const long long end = off0 + (long long)rows_src * cols_src;     // one past the last element
    auto dword = [&](long long k) -> uint32_t {                      // source dword k: elements 2k (low half) and 2k + 1
        const bool lo = 2 * k >= off0 && 2 * k < end, hi = 2 * k + 1 >= off0 && 2 * k + 1 < end;
        if (lo && hi) return base[k];
        const uint16_t* h = (const uint16_t*)base;
        return (lo ? (uint32_t)h[2 * k] : 0u) | (hi ? (uint32_t)h[2 * k + 1] << 16 : 0u);
    };
    const int col = 2 * i;
    auto one = [&](int row) -> uint32_t {                            // guarded form: any row, any position in the array
        uint32_t v = 0;
        if (row < rows_src && col < cols_src) {
            const long long f = off0 + (long long)row * cols_src + col;
            const long long k = f >> 1;
            if (f & 1) v = (dword(k) >> 16) | (dword(k + 1) << 16);
            else v = dword(k);
            if (col + 1 >= cols_src) v &= 0xFFFFu;
        }
        return v;
    };
    // four rows per step with all eight loads issued before the first use (a row is one dword per thread: the kernel is bound
    // by memory latency unless several rows are in flight); rows whose dwords k and k + 1 lie strictly inside the array only
    const int step = gridDim.y;
    int row = blockIdx.y;
    if (row == 0) { dst[i] = one(0); row += step; }
    const uint32_t keep = col + 1 >= cols_src ? 0xFFFFu : 0xFFFFFFFFu;
    if (col < cols_src && cols_src >= 8) {
        for (; (long long)row + 3LL * step < (long long)rows_src - 1; row += 4 * step) {
            uint32_t d0[4], d1[4];
            long long f[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                f[u] = off0 + (long long)(row + u * step) * cols_src + col;
                d0[u] = base[f[u] >> 1];
                d1[u] = base[(f[u] >> 1) + 1];
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const uint32_t v = (f[u] & 1) ? (d0[u] >> 16) | (d1[u] << 16) : d0[u];
                dst[(long long)(row + u * step) * per_row + i] = v & keep;
            }
        }
    }
    for (; row < rows_dst; row += step) dst[(long long)row * per_row + i] = one(row);
}

// 4-byte elements: one thread per element of a dst row, four rows in flight; grid = (ceil(cols_dst / 256), rows).
__global__ __launch_bounds__(256) void pad_rows32_kernel(const uint32_t* __restrict__ src, uint32_t* __restrict__ dst, int rows_src, int cols_src,
                                                         int rows_dst, int cols_dst)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= cols_dst) return;
    const int step = gridDim.y;
    int row = blockIdx.y;
    if (i < cols_src) {
        for (; (long long)row + 3LL * step < rows_src; row += 4 * step) {
            uint32_t d[4];
#pragma unroll
            for (int u = 0; u < 4; u++) d[u] = src[(long long)(row + u * step) * cols_src + i];
#pragma unroll
            for (int u = 0; u < 4; u++) dst[(long long)(row + u * step) * cols_dst + i] = d[u];
        }
    }
    for (; row < rows_dst; row += step) dst[(long long)row * cols_dst + i] = (row < rows_src && i < cols_src) ? src[(long long)row * cols_src + i] : 0u;
}
#endif

// dst [rows, cols] (dense, any row alignment, dst itself 16-byte aligned) <- the first cols columns of src [rows, cols_src]:
// one thread per 16-byte chunk of the flat destination; the last, partial chunk is stored by elements.
template <typename E>
__global__ __launch_bounds__(256) void unpad_rows_kernel(const E* __restrict__ src, E* __restrict__ dst, long long rows, int cols, int cols_src)
{
    constexpr int PER = 16 / (int)sizeof(E);
    typedef E Vec __attribute__((ext_vector_type(PER)));
    const long long total = rows * cols;
    const long long chunks = (total + PER - 1) / PER;
    const long long stride = (long long)gridDim.x * blockDim.x;
    for (long long g = (long long)blockIdx.x * blockDim.x + threadIdx.x; g < chunks; g += stride) {
        const long long f0 = g * PER;
        long long row = f0 / cols;
        int col = (int)(f0 - row * cols);
        Vec v;
#pragma unroll
        for (int e = 0; e < PER; e++) {
            v[e] = f0 + e < total ? src[row * cols_src + col] : (E)0;
            if (++col == cols) { col = 0; row++; }
        }
        if (f0 + PER <= total) *(Vec*)(dst + f0) = v;
        else for (int e = 0; e < PER && f0 + e < total; e++) dst[f0 + e] = v[e];
    }
}

// esize 2 or 4
hipError_t pad_rows(hipStream_t stream, const void* src, void* dst, int rows_src, int cols_src, int rows_dst, int cols_dst, int esize);
hipError_t unpad_rows(hipStream_t stream, const void* src, void* dst, long long rows, int cols, int cols_src, int esize);

#if AIDN_GEMM_PART == 0
static unsigned copy_grid(long long chunks)
{
    const long long wg = (chunks + 255) / 256;
    return (unsigned)(wg > 256 * 16 ? 256 * 16 : wg < 1 ? 1 : wg);
}
hipError_t pad_rows(hipStream_t stream, const void* src, void* dst, int rows_src, int cols_src, int rows_dst, int cols_dst, int esize)
{
    const long long chunks = (long long)rows_dst * (cols_dst / (16 / esize));
    if (esize == 2 && cols_dst >= 256) {
        const unsigned gy = (unsigned)((rows_dst + 7) / 8 < 8192 ? (rows_dst + 7) / 8 : 8192);      // about eight rows per thread
        hipLaunchKernelGGL(pad_rows16_kernel, dim3((unsigned)((cols_dst / 2 + 255) / 256), gy), dim3(256), 0, stream, (const uint16_t*)src, (uint32_t*)dst, rows_src, cols_src, rows_dst, cols_dst);
    } else if (esize == 2) hipLaunchKernelGGL((pad_rows_kernel<uint16_t>), dim3(copy_grid(chunks)), dim3(256), 0, stream, (const uint16_t*)src, (uint16_t*)dst, rows_src, cols_src, rows_dst, cols_dst);
    else if (cols_dst >= 128) {
        const unsigned gy = (unsigned)((rows_dst + 7) / 8 < 8192 ? (rows_dst + 7) / 8 : 8192);
        hipLaunchKernelGGL(pad_rows32_kernel, dim3((unsigned)((cols_dst + 255) / 256), gy), dim3(256), 0, stream, (const uint32_t*)src, (uint32_t*)dst, rows_src, cols_src, rows_dst, cols_dst);
    } else hipLaunchKernelGGL((pad_rows_kernel<uint32_t>), dim3(copy_grid(chunks)), dim3(256), 0, stream, (const uint32_t*)src, (uint32_t*)dst, rows_src, cols_src, rows_dst, cols_dst);
    return hipGetLastError();
}
hipError_t unpad_rows(hipStream_t stream, const void* src, void* dst, long long rows, int cols, int cols_src, int esize)
{
    const long long chunks = (rows * cols + 16 / esize - 1) / (16 / esize);
    if (esize == 2) hipLaunchKernelGGL((unpad_rows_kernel<uint16_t>), dim3(copy_grid(chunks)), dim3(256), 0, stream, (const uint16_t*)src, (uint16_t*)dst, rows, cols, cols_src);
    else hipLaunchKernelGGL((unpad_rows_kernel<uint32_t>), dim3(copy_grid(chunks)), dim3(256), 0, stream, (const uint32_t*)src, (uint32_t*)dst, rows, cols, cols_src);
    return hipGetLastError();
}

// The largest need over the plans gemm_16 may take for these dimensions (the choice also depends on operand alignment; every
// plan checks its own need against the bytes it is handed).
size_t gemm_16_workspace_bytes(int M, int N, int K)
{
    PadPlan pl;
    const size_t inner = gemm_16_inner_workspace_bytes(M, N, K);
    if (pad16_plan(M, N, K, &pl) && pl.total > inner) return pl.total;
    return inner;
}
// Pre-packed B (the caller keeps it): B [K,N] zero-padded to [Kp, Np] -- the copy that an unaligned product otherwise makes on every
// call, made once.  An aligned weight is packed the same way (its K and N padded to whole tiles).
size_t gemm_16_packed_b_bytes(int N, int K)
{
    PadPlan pl;
    if (N <= 0 || K <= 0 || !pad16_layout(1, N, K, &pl)) return 0;
    return (size_t)pl.Kp * pl.Np * 2;
}
hipError_t gemm_16_pack_b(hipStream_t stream, const uint16_t* B, int K, int N, void* packed)
{
    PadPlan pl;
    if (!pad16_layout(1, N, K, &pl) || !aligned16(packed)) return hipErrorInvalidValue;
    return pad_rows(stream, B, packed, K, N, pl.Kp, pl.Np, 2);
}
size_t gemm_16_packed_workspace_bytes(int M, int N, int K)
{
    PadPlan pl;
    return pad16_layout(M, N, K, &pl) ? pl.total : 0;
}
#endif

template <typename T, typename OutT>
static hipError_t launch_skinny(const GemmArgs& g, hipStream_t stream, float* ws, const RopeEpilogue* rope = nullptr)
{
    int ks;
    // more than 64 column slabs over a K of at most 4096 (16 x 28672 x 8192 went 77 -> 88 us): the three-stage form, two workgroups per CU (a workgroup's first memory round trip and its last
    // tiles run under the other's stream: 32 x 11008 x 4096 24.5 -> 22.9 us, 32 x 128256 x 4096 193 -> 187 us); with fewer slabs the
    // K ranges of that plan get too short (32 x 4096 x 4096 12.3 -> 14.1 us) and the seven-stage form, one per CU, stays
    const bool three = g.N / 128 > 64 && g.K <= 4096;
    const int kper = 64 * skinny_plan(g.N / 128, g.K / 64, &ks, three ? 2 : 1);
    if (three) {
        constexpr int smem = 3 * (32 * 128 + 64 * 256);
        static unsigned long long attr_done3 = 0;
        if (hipError_t e0 = ensure_dynamic_smem((const void*)gemm_skinny_kernel<T, 3>, smem, &attr_done3)) return e0;
            hipLaunchKernelGGL((gemm_skinny_kernel<T, 3>), dim3((unsigned)(g.N / 128), (unsigned)ks), dim3(256), smem, stream, g, ws, ks, kper);
    } else {
        constexpr int smem = SKINNY_STAGES * (32 * 128 + 64 * 256);
        static unsigned long long attr_done = 0;
        if (hipError_t e0 = ensure_dynamic_smem((const void*)gemm_skinny_kernel<T, SKINNY_STAGES>, smem, &attr_done)) return e0;
        hipLaunchKernelGGL((gemm_skinny_kernel<T, SKINNY_STAGES>), dim3((unsigned)(g.N / 128), (unsigned)ks), dim3(256), smem, stream, g, ws, ks, kper);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    long long total = (long long)g.M * g.N;
    unsigned grid = (unsigned)((total + 255) / 256);
    if constexpr (!std::is_same<OutT, float>::value) {
        if (rope) {
            grid = (unsigned)((total / 2 + 255) / 256);
            hipLaunchKernelGGL((skinny_reduce_rope_kernel<OutT>), dim3(grid), dim3(256), 0, stream, ws, (uint16_t*)g.C, g.M, g.N, ks, *rope);
            return hipGetLastError();
        }
    }
    hipLaunchKernelGGL((skinny_reduce_kernel<OutT>), dim3(grid), dim3(256), 0, stream, ws, g.C, g.M, g.N, ks, g.bias, g.act, g.act_param,
                       1.0f, 0.0f);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------------------------
// Small-M fp32 path (M <= 8, B stored [K,N] as fp32 or as fp16 weights): the GPU form of the N-parallel small-M GEMM.
// HBM-bound: B is read exactly once and nothing is staged, every lane owns four adjacent columns (one 16-byte load of a
// B row, 8 bytes for fp16 weights) and MR rows of accumulators; the A values of a k-row are the same for the whole wave
// and come through scalar loads.  grid = (ceil(N / 256), ksplit): the four waves of a workgroup take a quarter of the
// workgroup's K range each and are summed through LDS, the K ranges of different workgroups through an fp32 workspace that
// skinny_reduce_kernel sums in split order (deterministic) and finishes with alpha, beta, bias and activation.
template <int MR, bool B16, bool VEC>
__global__ __launch_bounds__(256) void gemm_smallm_kernel(const GemmArgs g, float* __restrict__ ws, int kper)
{
    __shared__ f32x4 red[3][MR][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n = blockIdx.x * 256 + lane * 4;
    const int ks = blockIdx.y;
    const int kb = ks * kper, ke = min(g.K, kb + kper);
    const int kq = ((ke - kb + 3) >> 2);
    const int k0 = min(ke, kb + wave * kq), k1 = min(ke, k0 + kq);
    const float* __restrict__ A = (const float*)g.A;
    const int nvalid = g.N - n;                       // columns this lane owns: min(4, nvalid), none if <= 0

    auto load_b = [&](int k) -> f32x4 {
        f32x4 r = {0.0f, 0.0f, 0.0f, 0.0f};
        if (nvalid <= 0) return r;
        if constexpr (B16) {
            const uint16_t* p = (const uint16_t*)g.B + (long long)k * g.ldb + n;
            if (VEC) {
                u32x2 w = __builtin_nontemporal_load((const u32x2*)p);
                r[0] = f16_bits_to_float(w[0] & 0xFFFFu); r[1] = f16_bits_to_float(w[0] >> 16);
                r[2] = f16_bits_to_float(w[1] & 0xFFFFu); r[3] = f16_bits_to_float(w[1] >> 16);
            } else {
#pragma unroll
                for (int e = 0; e < 4; e++) if (e < nvalid) r[e] = f16_bits_to_float(p[e]);
            }
        } else {
            const float* p = (const float*)g.B + (long long)k * g.ldb + n;
            if (VEC) r = __builtin_nontemporal_load((const f32x4*)p);      // B is read once per launch
            else {
#pragma unroll
                for (int e = 0; e < 4; e++) if (e < nvalid) r[e] = p[e];
            }
        }
        return r;
    };

    f32x4 acc[MR];
#pragma unroll
    for (int m = 0; m < MR; m++) acc[m] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    const float* arow[MR];
#pragma unroll
    for (int m = 0; m < MR; m++) arow[m] = A + (long long)min(m, g.M - 1) * g.lda;

    int k = k0;
    for (; k + 8 <= k1; k += 8) {
        f32x4 b[8];
#pragma unroll
        for (int u = 0; u < 8; u++) b[u] = load_b(k + u);
#pragma unroll
        for (int m = 0; m < MR; m++) {
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const float av = arow[m][k + u];
#pragma unroll
                for (int e = 0; e < 4; e++) acc[m][e] = fmaf(av, b[u][e], acc[m][e]);
            }
        }
    }
    for (; k < k1; k++) {
        const f32x4 b = load_b(k);
#pragma unroll
        for (int m = 0; m < MR; m++) {
            const float av = arow[m][k];
#pragma unroll
            for (int e = 0; e < 4; e++) acc[m][e] = fmaf(av, b[e], acc[m][e]);
        }
    }

    if (wave > 0) {
#pragma unroll
        for (int m = 0; m < MR; m++) red[wave - 1][m][lane] = acc[m];
    }
    __syncthreads();
    if (wave == 0 && nvalid > 0) {
#pragma unroll
        for (int m = 0; m < MR; m++) {
            if (m < g.M) {
                f32x4 v = acc[m];
#pragma unroll
                for (int w = 0; w < 3; w++) {
                    const f32x4 o = red[w][m][lane];
#pragma unroll
                    for (int e = 0; e < 4; e++) v[e] += o[e];
                }
                float* dst = ws + ((long long)ks * g.M + m) * g.N + n;
                if (VEC && (g.N & 3) == 0) *(f32x4*)dst = v;          // (rows of B may be padded beyond an N that is no multiple of 4)
                else {
#pragma unroll
                    for (int e = 0; e < 4; e++) if (e < nvalid) dst[e] = v[e];
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Skinny-M fp32 path: 9 <= M <= 32, B stored [K,N], N % 128 == 0, K % 32 == 0 -- the fp32 form of gemm_skinny_kernel.
// HBM-bound: B is read exactly once.  grid = (N / 128, KS); a workgroup streams a 128-column slab of B over its K range through
// a ring of NS (three: two workgroups per CU) 20 KB stages (32 k-rows of 512 bytes of B and 32 rows of 128 bytes of A per stage, five
// direct-to-LDS loads per wave and K-tile), each wave multiplies the 32 x 32 block of its 32 columns on the fp32 MFMA (a 64-row
// tile of the general kernel would spend three quarters of its matrix work on padding and run at a quarter of the memory rate)
// and stores the partial product for skinny_reduce_kernel.
//   B tile [32 k][512 B]: chunk c of row k at position c ^ (((k >> 2) & 1) << 3)   (32-bit reads; the lane halves read rows 4 apart)
//   A tile [32 m][128 B]: chunk c of row m at position c ^ ((m >> 1) & 7)          (b128 reads)
// The k index of MFMA step i of 8-k group j is 8 j + 4 h + i for both operands (h = lane half).
#if AIDN_GEMM_PART == 0
template <int NS>
__global__ __launch_bounds__(256, NS <= 3 ? 2 : 1) void gemm_skinny32_kernel(const GemmArgs g, float* __restrict__ ws, int ksplit, int kper)
{
    constexpr int BK = 32, AHEAD = NS - 1;
    constexpr int ABYTES = 32 * 128, BBYTES = BK * 512, STAGE = ABYTES + BBYTES;
    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];      // NS stages

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    const int n0 = blockIdx.x * 128;
    const int ks = blockIdx.y;
    const int kbeg = ks * kper;
    const int KT = min(kper, g.K - kbeg) / BK;            // the last range may be shorter
    const float* __restrict__ A = (const float*)g.A;
    const float* __restrict__ B = (const float*)g.B;

    // this wave's DMA per K-tile: 4 B wave-loads (k-rows 2w', 2w'+1 with w' = 4 wave + i) and A wave-load `wave` (rows 8 wave ..)
    const float* pb[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int row = 2 * (wave * 4 + i) + (lane >> 5), pos = lane & 31;
        pb[i] = B + (long long)(kbeg + row) * g.ldb + n0 + (pos ^ (((row >> 2) & 1) << 3)) * 4;
    }
    const float* pa;
    {
        const int row = 8 * wave + (lane >> 3), pos = lane & 7;
        const int grow = min(row, g.M - 1);
        pa = A + (long long)grow * g.lda + kbeg + (pos ^ ((row >> 1) & 7)) * 4;
    }
    auto issue_loads = [&](int kt, int stage) {
        unsigned char* as = smem + stage * STAGE;
        unsigned char* bs = as + ABYTES;
        dma16_to_lds(pa + kt * BK, as + wave * 1024);
#pragma unroll
        for (int i = 0; i < 4; i++) dma16_to_lds_stream(pb[i] + (long long)kt * BK * g.ldb, bs + (wave * 4 + i) * 1024);
    };

    const int a_off = l32 * 128, a_sw = (l32 >> 1) & 7;
    const int b_col = wave * 32 + l32;                  // column inside the slab

    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.0f;

    for (int kt = 0; kt < AHEAD && kt < KT; kt++) issue_loads(kt, kt);
    int stage = 0;
    for (int kt = 0; kt < KT; kt++) {
        // tiles kt+1 .. kt+AHEAD-1 (those that exist) are younger than tile kt: five loads per wave each
        switch (min(KT - 1 - kt, AHEAD - 1)) {
            case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
            case 1: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
            case 2: asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); break;
            case 3: asm volatile("s_waitcnt vmcnt(15)" ::: "memory"); break;
            case 4: asm volatile("s_waitcnt vmcnt(20)" ::: "memory"); break;
            default: asm volatile("s_waitcnt vmcnt(25)" ::: "memory"); break;
        }
        __syncthreads();            // everyone's part of tile kt has landed, and everyone has left tile kt-1
        if (kt + AHEAD < KT) issue_loads(kt + AHEAD, stage == 0 ? NS - 1 : stage - 1);      // into the stage tile kt-1 used
        const unsigned char* as = smem + stage * STAGE;
        const unsigned char* bs = as + ABYTES;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const u32x4 fa = *(const u32x4*)(as + a_off + (((2 * j + h) ^ a_sw) << 4));
            u32x4 fb;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = 8 * j + 4 * h + i;          // (row >> 2) & 1 == h
                fb[i] = *(const uint32_t*)(bs + row * 512 + ((((b_col >> 2) ^ (h << 3)) << 4) + (b_col & 3) * 4));
            }
            Mma32<float>::run(acc, fa, fb);
        }
        stage = stage + 1 == NS ? 0 : stage + 1;
    }

    const int col = n0 + b_col;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int row = acc_row(r, h);
        if (row < g.M) ws[((long long)ks * g.M + row) * g.N + col] = acc[r];
    }
}
#endif

[[maybe_unused]] static bool skinny32_applies(int M, int N, int K) { return M > 8 && M <= 32 && N % 128 == 0 && K % 32 == 0 && N >= 128; }

// The fp32 skinny kernel runs a three-stage ring, two workgroups per CU: a workgroup's first memory round trip and its last tiles
// run under the other's stream (against seven stages and one per CU: 16 x 8192 x 8192 57.3 -> 48.3 us, 16 x 28672 x 8192 204 -> 171 us,
// 16 x 11008 x 4096 50.3 -> 41.1 us, 16 x 4096 x 4096 20.1 -> 18.4 us).  K-tiles per range; *ks ranges.
#define SKINNY32_STAGES 3
[[maybe_unused]] static int skinny32_plan(int N, int K, int* ks) { return skinny_plan(N / 128, K / 32, ks, 2); }
[[maybe_unused]] static int skinny32_ksplit(int N, int K) { int ks; skinny32_plan(N, K, &ks); return ks; }

// fp32: estimated run time (microseconds) of the direct-to-LDS kernel with `tile` x `tile` tiles when K is cut into `ks` ranges
// that run as batches.  A CU works through its tiles at the same total rate whether it holds one or two at a time, so the time
// is (tiles of the busiest CU) x (MFMA time of one padded tile); per flop the 256 and 128 tiles run at about 0.88 and the 64
// tile at about 0.75 of the fp32 peak (614 GFLOP/s per CU).  K ranges add the pass that sums the fp32 partials.  The estimate
// reproduces what was measured where the choice matters (128 x 50304 x 768: 186 / 93 / 96 us estimated for the three tiles,
// 179 / 93 / 84 measured; 16 x 4096 x 4096 on 64 x 64 tiles: 73 estimated, 77 measured).
[[maybe_unused]] static double f32_time_us(int M, int N, int K, long long batch, int tile, int ks)
{
    const long long wg = (long long)((M + tile - 1) / tile) * ((N + tile - 1) / tile) * batch * ks;
    const double rounds = wg <= 2048 ? (double)((wg + 255) / 256) : (double)wg / 256.0 + 0.5;
    // the 64 x 64 tile comes close to the rate of the larger ones once several workgroups share a CU (3000 x 4096 x 4096: 3008 tiles
    // at 0.88 of the pipe; with operands beyond the caches its doubled traffic per flop costs a few per cent), and 0.75 with one
    // per CU, where a lone wave per SIMD overlaps nothing
    const double eff = tile == 64 ? (wg >= 1024 ? 0.85 : wg >= 512 ? 0.80 : 0.75) : 0.88;
    double tile_us = 2.0 * tile * tile * (double)(K / ks) / (0.614e6 * eff) + 1.5;
    // measured: the 128 x 128 instance with edge handling takes 922 us where the plain one takes 721 us on 768 tiles (M = 2945..3071
    // against 3072, N = K = 4096; one ragged row is enough), 3 % more on 256 tiles (M = 1023) and nothing extra on 1536 tiles.  Two
    // such workgroups share a CU; 512 tiles take 470 us with either instance, and the 256 tiles of the last round are then spread
    // one per CU (+250 us) or packed two per CU on half the chip (+450 us) -- the hardware dispatcher's placement, which came out
    // the second way for the edge instance; the 64 x 64 instance shows no such step
    if (tile == 128 && (M % 128 != 0 || N % 128 != 0)) tile_us *= wg > 512 && wg <= 1024 ? 1.25 : 1.03;
    double t = rounds * tile_us;
    if (ks > 1) t += 3.0 + (double)(ks + 2) * M * N * 4.0 / 3.0e6;
    return t;
}

// fp32 tile edge for a problem that is not split (256 only where the direct-to-LDS kernel may run it)
[[maybe_unused]] static int f32_tile(int M, int N, int K, long long batch, bool allow256)
{
    int best = 128;
    double bt = f32_time_us(M, N, K, batch, 128, 1);
    const double t64 = f32_time_us(M, N, K, batch, 64, 1);
    if (t64 < bt) { bt = t64; best = 64; }
    if (allow256 && f32_time_us(M, N, K, batch, 256, 1) <= bt) best = 256;
    return best;
}

// fp32 split-K: number of K ranges (1 = none) that the estimate prefers for a single product.  Ranges are equal multiples of 32
// of at least 256; a split must beat the unsplit estimate by 15 % to be taken (it costs a second launch and workspace).
[[maybe_unused]] static int splitk32_ranges(int M, int N, int K)
{
    if (K < 1024 || K % 32 != 0) return 1;
    double best = f32_time_us(M, N, K, 1, f32_tile(M, N, K, 1, true), 1) * 0.95;
    int best_ks = 1;
    const int cand[7] = {2, 3, 4, 6, 8, 12, 16};
    for (int i = 0; i < 7; i++) {
        const int ks = cand[i];
        if (K % (ks * 32) != 0 || K / ks < 256) continue;
        const double t = std::min(f32_time_us(M, N, K, 1, 128, ks), f32_time_us(M, N, K, 1, 64, ks));
        if (t < best) { best = t; best_ks = ks; }
    }
    return best_ks;
}

static bool smallm_applies(int M, int N, int K) { return M >= 1 && M <= 8 && (long long)N * K >= 4096; }

// K range of one workgroup: about 1024 workgroups, at least 128 k-rows each (32 per wave), a multiple of 32
static int smallm_kper(int N, int K)
{
    const int colblocks = (N + 255) / 256;
    int ks = (1024 + colblocks - 1) / colblocks;
    int kper = (K + ks - 1) / ks;
    if (kper < 128) kper = 128;
    kper = (kper + 31) / 32 * 32;
    // K ranges that start a multiple of 4 MiB apart put the workgroups of a column block on the same memory channels
    // (1 x 8192 x 8192: 60 us with 256-row ranges, 8 MiB apart, against 43-48 us with any other size)
    for (int tries = 0; tries < 64 && ((long long)kper * N * 4) % (1LL << 22) == 0; tries++) kper += 8;   // (bounded: a very wide N aliases at every multiple of 32)
    return kper;
}

#if AIDN_GEMM_PART == 0
size_t gemm_smallm_workspace_bytes(int M, int N, int K)
{
    if (!smallm_applies(M, N, K)) return 0;
    const int kper = smallm_kper(N, K);
    return (size_t)((K + kper - 1) / kper) * M * N * sizeof(float);
}
// fp32 problems whose rows are not whole 16-byte chunks (K, or N with B [K,N], not a multiple of 4): zero-padded copies of A and B
// in the workspace (K up to a multiple of 32, N up to a multiple of 4) feed the direct-to-LDS kernel, whose element stores put the N
// real columns straight into the caller's C.  Same sums as the plain product: the padding contributes exact zeros.
struct Pad32Plan { int Np, Kp; size_t a_off, b_off, total; };
static bool pad32_layout(int M, int N, int K, int transB, Pad32Plan* pl)
{
    pl->Kp = (K + 31) / 32 * 32;
    pl->Np = transB ? N : (N + 3) / 4 * 4;
    if (pl->Kp >= (1 << 21) || pl->Np >= (1 << 21)) return false;
    auto up = [](size_t b) { return (b + 255) & ~(size_t)255; };
    pl->a_off = 0;
    pl->b_off = up((size_t)M * pl->Kp * 4);
    pl->total = pl->b_off + up((size_t)(transB ? N : pl->Kp) * (transB ? pl->Kp : pl->Np) * 4);
    return pl->total <= ((size_t)4 << 30);
}
static bool pad32_plan(int M, int N, int K, int transB, Pad32Plan* pl)
{
    if (K % 4 == 0 && (transB || N % 4 == 0)) return false;
    if (N < 16 || (double)M * N * K < (double)(1 << 21)) return false;
    if (M <= 512 && K <= 1024) return false;          // as for 16-bit: the general kernel reads the rows in place
    return pad32_layout(M, N, K, transB, pl);
}

// Pre-packed fp32 B (the caller keeps it): [K,N] zero-padded to [Kp, Np], or [N,K] to [N, Kp] -- the GPU form of the reference's
// cached packed weight operand (SimdGemm.SgemmWithCachedB / PrePackedB): packed once, the product is that of the plain call.
size_t gemm_f32_packed_b_bytes(int N, int K, int transB)
{
    Pad32Plan pl;
    if (N <= 0 || K <= 0 || !pad32_layout(1, N, K, transB, &pl)) return 0;
    return (size_t)(transB ? N : pl.Kp) * (transB ? pl.Kp : pl.Np) * 4;
}
hipError_t gemm_f32_pack_b(hipStream_t stream, const float* B, int K, int N, int transB, void* packed)
{
    Pad32Plan pl;
    if (!pad32_layout(1, N, K, transB, &pl) || !aligned16(packed)) return hipErrorInvalidValue;
    return transB ? pad_rows(stream, B, packed, N, K, N, pl.Kp, 4) : pad_rows(stream, B, packed, K, N, pl.Kp, pl.Np, 4);
}
size_t gemm_f32_packed_workspace_bytes(int M, int N, int K, int transB)
{
    Pad32Plan pl;
    if (!pad32_layout(M, N, K, transB, &pl)) return 0;
    const size_t small = !transB && smallm_applies(M, N, K) ? gemm_smallm_workspace_bytes(M, N, K) : 0;
    return pl.b_off > small ? pl.b_off : small;                       // the padded copy of A, or the small-M partials
}

// The largest need over every plan gemm_f32 may take for these dimensions: which one it takes also depends on the alignment of
// the operands, which the sizing does not see, and every plan checks its own need against the bytes it is handed.
size_t gemm_f32_workspace_bytes(int M, int N, int K, int transB)
{
    size_t need = 0;
    auto upto = [&](size_t n) { if (n > need) need = n; };
    Pad32Plan pl;
    if (pad32_plan(M, N, K, transB, &pl)) upto(pl.total);
    if (!transB && smallm_applies(M, N, K)) upto(gemm_smallm_workspace_bytes(M, N, K));
    if (!transB && skinny32_applies(M, N, K)) upto((size_t)skinny32_ksplit(N, K) * M * N * sizeof(float));
    const int ks = splitk32_ranges(M, N, K);
    if (ks > 1) upto((size_t)ks * M * N * sizeof(float));
    return need;
}
#endif

template <bool B16>
static hipError_t launch_smallm(const GemmArgs& g, hipStream_t stream, float* ws)
{
    const int kper = smallm_kper(g.N, g.K);
    const int ks = (g.K + kper - 1) / kper;
    // whole 16-byte loads of B: rows in 16-byte steps that hold every chunk a lane may touch (N a multiple of 4, or rows padded to one)
    const bool vec = (g.N % 4 == 0 || g.ldb >= (g.N + 3) / 4 * 4) && g.ldb % 4 == 0 && (((uintptr_t)g.B) & (B16 ? 7u : 15u)) == 0;
    const dim3 grid((unsigned)((g.N + 255) / 256), (unsigned)ks);
    const int mr = g.M <= 1 ? 1 : g.M <= 2 ? 2 : g.M <= 4 ? 4 : 8;
#define AIDN_SMALLM(MR_)                                                                                               \
    do {                                                                                                               \
        if (vec) hipLaunchKernelGGL((gemm_smallm_kernel<MR_, B16, true>), grid, dim3(256), 0, stream, g, ws, kper);     \
        else hipLaunchKernelGGL((gemm_smallm_kernel<MR_, B16, false>), grid, dim3(256), 0, stream, g, ws, kper);        \
    } while (0)
    if (mr == 1) AIDN_SMALLM(1);
    else if (mr == 2) AIDN_SMALLM(2);
    else if (mr == 4) AIDN_SMALLM(4);
    else AIDN_SMALLM(8);
#undef AIDN_SMALLM
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const long long total = (long long)g.M * g.N;
    hipLaunchKernelGGL((skinny_reduce_kernel<float>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, ws, g.C, g.M, g.N, ks,
                       g.bias, g.act, g.act_param, g.alpha, g.beta);
    return hipGetLastError();
}

// ------------------------------------------------------------------ host side
template <typename T, typename OutT, int BM, int BN, int WM, int WN, bool TRANSB, bool VEC, bool CHECK, int KS = 1, bool B16 = false>
static hipError_t launch_gemm(GemmArgs g, int batch, hipStream_t stream)
{
    auto kern = gemm_kernel<T, OutT, BM, BN, WM, WN, TRANSB, VEC, CHECK, KS, B16>;
    constexpr int tiles_smem = 2 * (BM + BN) * gemm_row_pitch(BM, BN), merge_smem = KS == 2 ? BM * BN * 4 : 0;
    constexpr int smem = tiles_smem > merge_smem ? tiles_smem : merge_smem;
    static unsigned long long attr_done = 0;
    if (hipError_t e = ensure_dynamic_smem((const void*)kern, smem, &attr_done)) return e;
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    dim3 grid((unsigned)(g.tiles_m * g.tiles_n), 1, (unsigned)batch);
    hipLaunchKernelGGL(kern, grid, dim3(WM * WN * KS * 64), smem, stream, g);
    return hipGetLastError();
}



// 128 x 128 or 64 x 64 tile; rel64 = efficiency per flop of the smaller tile relative to the larger one when both load the
// CUs equally well (measured: about 0.85 for fp32, 0.55 for the 16-bit types).
static int choose_tile(long long tiles128, long long tiles64, double rel64)
{
    return cu_fill(tiles128) >= rel64 * cu_fill(tiles64) ? 128 : 64;
}

// what the 16 x 16 x 32 kernel needs beyond whole tiles: 16-byte aligned operand rows, C rows and bias, and the plain product
template <typename OutT>
static bool dl16_applies(const GemmArgs& g)
{
    const int OB = Elem<OutT>::BYTES;
    return aligned16(g.A) && aligned16(g.B) && g.lda % 8 == 0 && g.ldb % 8 == 0 && g.sA % 8 == 0 && g.sB % 8 == 0 &&
           g.lda < (1 << 21) && g.ldb < (1 << 21) &&
           aligned16(g.C) && ((long long)g.ldc * OB) % 16 == 0 && (g.sC * OB) % 16 == 0 && (g.bias == nullptr || aligned16(g.bias)) &&
           g.alpha == 1.0f && g.beta == 0.0f;
}

// Tile width (in 64-column units: 4, 3 or 2) of the 16 x 16 x 32 kernel for a 16-bit problem with K % 64 == 0 (any M), or 0
// when none of the widths divides N or the 128 x 128 / 64 x 64 tiles of the 32 x 32 x 16 kernel are expected to finish earlier.
// Every candidate is scored as (how evenly its tiles load the 256 CUs) x (its rate per flop relative to the 256 x 256 tile): a
// narrower tile moves more A bytes per flop (and the 256 x 128 one wastes half of its B loads); the 128 x 128 tile runs at about
// 0.55 and the 64 x 64 tile at about 0.45 of the 256 x 256 rate (2048^3: 128 tiles of 256 x 128 take 36 us, 256 tiles of 128 x 128 29 us).
#define DL16_HALF_EFF 0.7
#define DL16_HALF2_EFF 0.82
static int dl16_width(int M, int N, int K, int batch, double* score_out)
{
    if (score_out) *score_out = 0.0;
    if (K % 64 != 0) return 0;
    // M may be ragged (the last tile row is partial: clamped loads, guarded stores); the rows a tile height pads count as waste
    const long long tm256 = (M + 255) / 256, tm128 = (M + 127) / 128, tm64 = (M + 63) / 64;
    const double use256 = (double)M / (double)(tm256 * 256), use128 = (double)M / (double)(tm128 * 128), use64 = (double)M / (double)(tm64 * 64);
    const int widths[3] = {4, 3, 2};
    const double eff[3] = {1.0, 0.94, 0.8};
    int best = 0;
    double best_score = 0.0;
    for (int i = 0; i < 3; i++) {
        const int bn = 64 * widths[i];
        if (N % bn != 0) continue;
        const long long t = tm256 * (N / bn) * batch;
        const double score = cu_fill(t) * eff[i] * use256;
        if (score > best_score) { best_score = score; best = widths[i]; }
    }
    const long long t128 = tm128 * ((N + 127) / 128) * batch;
    const long long t64 = tm64 * ((N + 63) / 64) * batch;
    // the 128 x 128 tile of this kernel (code 1): whole column tiles only
    if (N % 128 == 0 && DL16_HALF_EFF * cu_fill(t128) * use128 > best_score) { best_score = DL16_HALF_EFF * cu_fill(t128) * use128; best = 1; }
    // the same tile on a two-stage ring, two workgroups per CU (code 5): with more tiles than CUs and a K of at most 6144 one
    // workgroup's first loads, barrier waits and store phase run under the other's MFMAs (8192 x 768 x 3072 50.4 -> 41.8 us,
    // 512 x 12288 x 4096 64.8 -> 54.4 us, 384 x 13824 x 5120 79.8 -> 65.8 us); one tile per CU (2048^3 20.7 -> 27.6 us) and long K
    // (384 x 28672 x 8192 228 -> 265 us) need the deeper ring
    // (beyond one round of 512 resident workgroups only when the last round is nearly full: a workgroup alone on its CU has nothing
    // to hide the two-stage ring's waits behind -- 3000 x 4096 x 4096, 768 tiles: 83 -> 106 us)
    const double fill2 = (double)t128 / (double)(((t128 + 511) / 512) * 512);
    if (N % 128 == 0 && t128 > 256 && K <= 6144 && (t128 <= 512 || fill2 >= 0.85)) {
        const double s2 = DL16_HALF2_EFF * (t128 <= 512 ? cu_fill(t128) : fill2) * use128;
        if (s2 > best_score) { best_score = s2; best = 5; }
    }
    const double s128 = 0.55 * cu_fill(t128) * use128, s64 = 0.45 * cu_fill(t64) * use64;
    if (score_out) *score_out = best_score > s128 ? (best_score > s64 ? best_score : s64) : (s128 > s64 ? s128 : s64);
    if (s128 > best_score || s64 > best_score) return 0;
    return best;
}

// Kernel and tile choice: the 256 x 256 direct-to-LDS kernel for 16-bit B[K,N] problems with at least 128 such tiles,
// otherwise the general kernel with the 128 x 128 or 64 x 64 tile (choose_tile), in its branch-free instance when the
// operands are 16-byte aligned and the K-tile divides K.
template <typename T, typename OutT, bool TRANSB>
static hipError_t dispatch_gemm(const GemmArgs& g, int batch, hipStream_t stream, int force_tile)
{
    constexpr int E = Elem<T>::PER16;
    const bool vec = aligned16(g.A) && aligned16(g.B) && g.lda % E == 0 && g.ldb % E == 0 && g.K % E == 0 &&
                     (TRANSB || g.N % E == 0) && g.sA % E == 0 && g.sB % E == 0;
    auto tiles = [&](int bm, int bn) { return (long long)((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn) * batch; };
    int tile = force_tile;
    if (tile == 0) {
        if constexpr (!TRANSB || E == 4) {
            // the direct-to-LDS kernel: rows of A and B in whole 16-byte chunks, leading dimensions within the 32-bit lane
            // offsets of its loads; M, N and K may be ragged
            if (vec && g.lda < (1 << 21) && g.ldb < (1 << 21) && (Elem<OutT>::BYTES == 4 || (g.alpha == 1.0f && g.beta == 0.0f))) {
                // 16-bit: the 256 x 256 tile moves half the bytes per flop of the 128 x 128 one and wins from half a chip of
                // tiles on; fp32 runs both at about the same rate per flop, so there the better CU load decides
                if constexpr (E == 8 && !TRANSB) {
                    if (dl16_applies<OutT>(g)) {
                        const int w = dl16_width(g.M, g.N, g.K, batch);
                        if (w == 4) return launch_gemm_dl16<T, OutT, 4>(g, batch, stream);
                        if (w == 3) return launch_gemm_dl16<T, OutT, 3>(g, batch, stream);
                        if (w == 2) return launch_gemm_dl16<T, OutT, 2>(g, batch, stream);
                        if (w == 1) return launch_gemm_dl16<T, OutT, 2, true>(g, batch, stream);
                        if (w == 5) return launch_gemm_dl16<T, OutT, 2, true, 2>(g, batch, stream);
                    }
                }
                if constexpr (E == 4) {
                    // fp32 runs every tile at about the same rate per flop: the estimated time, padding included, decides
                    const int t = f32_tile(g.M, g.N, g.K, batch, true);
                    tile = t == 256 ? 256 : t == 128 ? 129 : 65;
                } else {
                    const long long t256 = tiles(256, 256), t128 = tiles(128, 128);
                    // (16-bit, ragged or unaligned for the 16 x 16 x 32 kernel: the 256 x 256 tile of this kernel when it scores best)
                    const bool big = t256 >= 128 && cu_fill(t256) >= 0.55 * cu_fill(t128);
                    // otherwise the same kernel with 128 x 128 or 64 x 64 tiles (codes 129, 65), whichever loads the CUs better; per
                    // flop the 64 x 64 instance runs at about 0.8 of the 128 x 128 one
                    if (big) tile = 256;
                    else tile = choose_tile(t128, tiles(64, 64), 0.8) == 128 ? 129 : 65;
                }
            }
        }
        // (at most 64 rows: bound by the stream of B, which more and smaller workgroups keep fuller)
        if (tile == 0) tile = g.M <= 64 ? 64 : E == 4 ? f32_tile(g.M, g.N, g.K, batch, false) : choose_tile(tiles(128, 128), tiles(64, 64), 0.55);
    }
    if constexpr (E == 8 && !TRANSB) {
        if (tile == 192 || tile == 193) {                 // 256 x 192 / 256 x 128 tiles of the 16 x 16 x 32 kernel (whole tiles only)
            const int bn = tile == 192 ? 192 : 128;
            if (!(g.N % bn == 0 && g.K % 64 == 0 && dl16_applies<OutT>(g))) return hipErrorInvalidValue;
            return tile == 192 ? launch_gemm_dl16<T, OutT, 3>(g, batch, stream) : launch_gemm_dl16<T, OutT, 2>(g, batch, stream);
        }
    }
    if constexpr (E == 8 && !TRANSB) {
        if (tile == 131) {                                // the same on the two-stage ring (two workgroups per CU)
            if (!(g.N % 128 == 0 && g.K % 64 == 0 && dl16_applies<OutT>(g))) return hipErrorInvalidValue;
            return launch_gemm_dl16<T, OutT, 2, true, 2>(g, batch, stream);
        }
        if (tile == 130) {                                // 128 x 128 tiles of the 16 x 16 x 32 kernel (whole tiles only)
            if (!(g.N % 128 == 0 && g.K % 64 == 0 && dl16_applies<OutT>(g))) return hipErrorInvalidValue;
            return launch_gemm_dl16<T, OutT, 2, true>(g, batch, stream);
        }
    }
    if (tile == 192 || tile == 193 || tile == 130 || tile == 131) return hipErrorInvalidValue;
    if constexpr (E == 4 || !TRANSB) {
        if (tile == 65) {                                 // 64 x 64 tiles on the direct-to-LDS kernel
            if (!(vec && (TRANSB || g.N >= E) && g.lda < (1 << 21) && g.ldb < (1 << 21))) return hipErrorInvalidValue;
            if (Elem<OutT>::BYTES != 4 && (g.alpha != 1.0f || g.beta != 0.0f)) return hipErrorInvalidValue;
            const bool exact_fit = g.M % 64 == 0 && g.N % 64 == 0 && g.K % (8 * E) == 0 && g.c_cols == 0;
            if constexpr (E == 4 && !TRANSB) {
                // about one tile per CU: the eight-wave form (two k-step groups), so that every SIMD has a second wave to switch to
                if (exact_fit && tiles(64, 64) <= 512) return launch_gemm_dl<T, OutT, false, 64, TRANSB, 2>(g, batch, stream);
            }
            return exact_fit ? launch_gemm_dl<T, OutT, false, 64, TRANSB>(g, batch, stream) : launch_gemm_dl<T, OutT, true, 64, TRANSB>(g, batch, stream);
        }
    }
    if (tile == 65) tile = 64;
    if constexpr (!TRANSB || E == 4) {
        if (tile == 256 || tile == 129) {
            if (!(vec && (TRANSB || g.N >= E) && g.lda < (1 << 21) && g.ldb < (1 << 21))) return hipErrorInvalidValue;
            if (Elem<OutT>::BYTES != 4 && (g.alpha != 1.0f || g.beta != 0.0f)) return hipErrorInvalidValue;
            const int edge = tile == 256 ? 256 : 128;
            const bool exact_fit = g.M % edge == 0 && g.N % edge == 0 && g.K % (8 * E) == 0 && g.c_cols == 0;
            // (bf16 output with ragged edges on the 256 x 256 tile: that one instance does not fit the register file -- the
            // compiler moves accumulators to scratch memory -- so such problems take the 128 x 128 tile)
            constexpr bool kSpills256Edge = std::is_same<T, bf16_t>::value && std::is_same<OutT, bf16_t>::value;
            if constexpr (E == 8 && !TRANSB) {
                // 16-bit, whole tiles: the 16 x 16 x 32 kernel (its stores and bias loads are 16-byte vectors: C rows and the bias
                // must be 16-byte aligned; it computes act(A B + bias), so alpha = 1 and beta = 0)
                if (tile == 256 && exact_fit && dl16_applies<OutT>(g)) return launch_gemm_dl16<T, OutT, 4>(g, batch, stream);
            }
            if (tile == 256 && exact_fit) return launch_gemm_dl<T, OutT, false, 256, TRANSB>(g, batch, stream);
            if constexpr (!kSpills256Edge) {
                if (tile == 256) return launch_gemm_dl<T, OutT, true, 256, TRANSB>(g, batch, stream);
            }
            return exact_fit ? launch_gemm_dl<T, OutT, false, 128, TRANSB>(g, batch, stream) : launch_gemm_dl<T, OutT, true, 128, TRANSB>(g, batch, stream);
        }
    }
    if (tile == 129) tile = 128;
    if (g.c_cols > 0) return hipErrorInvalidValue;        // only the direct-to-LDS kernels above know that C is narrower than N
    // 16-byte aligned operands whose K the K-tile divides take the instance without bounds checks in its loop (no zero fill
    // is needed; rows and column blocks past the end are clamped loads whose products are never stored)
    auto exact = [&](int bt) { return vec && g.N >= E && g.K % (gemm_k_chunks(bt, bt) * E) == 0; };
    if (tile == 128) {
        if (exact(128)) return launch_gemm<T, OutT, 128, 128, 2, 2, TRANSB, true, false>(g, batch, stream);
        if (vec) return launch_gemm<T, OutT, 128, 128, 2, 2, TRANSB, true, true>(g, batch, stream);
        return launch_gemm<T, OutT, 128, 128, 2, 2, TRANSB, false, true>(g, batch, stream);
    }
    if (tile == 64) {
        // at most about one 64 x 64 tile per CU: split every K-tile between two wave groups so each SIMD still holds two waves
        if (vec && tiles(64, 64) <= 320 && g.K >= 4 * 16 * E) {
            if (exact(64)) return launch_gemm<T, OutT, 64, 64, 2, 2, TRANSB, true, false, 2>(g, batch, stream);
            return launch_gemm<T, OutT, 64, 64, 2, 2, TRANSB, true, true, 2>(g, batch, stream);
        }
        if (exact(64)) return launch_gemm<T, OutT, 64, 64, 2, 2, TRANSB, true, false>(g, batch, stream);
        if (vec) return launch_gemm<T, OutT, 64, 64, 2, 2, TRANSB, true, true>(g, batch, stream);
        return launch_gemm<T, OutT, 64, 64, 2, 2, TRANSB, false, true>(g, batch, stream);
    }
    return hipErrorInvalidValue;
}

#if AIDN_GEMM_PART == 0
hipError_t gemm_f32(hipStream_t stream, const float* A, const float* B, float* C, int M, int N, int K,
                    float alpha, float beta, int transB, int batch, long long sA, long long sB, long long sC,
                    int force_tile, const float* bias, int act, float act_param, void* workspace, const float* Bpre,
                    size_t workspace_bytes)
{
    GemmArgs g{A, B, C, M, N, K, K, transB ? K : N, N, sA, sB, sC, alpha, beta, 0, 0, bias, act, act_param};
    if (!workspace) workspace_bytes = 0;
    // every plan below that writes to the workspace first holds its own need against the bytes handed in, and is passed over
    // (down to the tiled kernels, which need none) when they do not suffice
    const bool smallm_fits = workspace && smallm_applies(M, N, K) && gemm_smallm_workspace_bytes(M, N, K) <= workspace_bytes;
    if (!Bpre && force_tile == 0 && smallm_fits && !transB && batch == 1)
        return launch_smallm<false>(g, stream, (float*)workspace);
    // Bpre: B already packed by gemm_f32_pack_b (B itself is then not read); such a call always takes the padded shapes
    Pad32Plan pl;
    if (Bpre && !transB && batch == 1 && smallm_fits && aligned16(Bpre) && pad32_layout(M, N, K, 0, &pl)) {
        GemmArgs gs = g;
        gs.B = Bpre; gs.ldb = pl.Np;                 // the padded rows; only the first K of them are read
        return launch_smallm<false>(gs, stream, (float*)workspace);
    }
    if (Bpre && !(batch == 1 && aligned16(Bpre) && pad32_layout(M, N, K, transB, &pl) &&
                  (pl.Kp == K ? aligned16(A) : (workspace && aligned16(workspace) && pl.b_off <= workspace_bytes))))
        return hipErrorInvalidValue;
    if (Bpre || (force_tile == 0 && workspace && batch == 1 && aligned16(workspace) && pad32_plan(M, N, K, transB, &pl) && pl.total <= workspace_bytes &&
                 (pl.Kp != K || aligned16(A)))) {
        unsigned char* w = (unsigned char*)workspace;
        const float* Ap = A;
        if (pl.Kp != K) {
            if (hipError_t e = pad_rows(stream, A, w + pl.a_off, M, K, M, pl.Kp, 4)) return e;
            Ap = (const float*)(w + pl.a_off);
        }
        const void* Bp = Bpre;
        if (!Bpre) {
            if (hipError_t e = transB ? pad_rows(stream, B, w + pl.b_off, N, K, N, pl.Kp, 4) : pad_rows(stream, B, w + pl.b_off, K, N, pl.Kp, pl.Np, 4)) return e;
            Bp = w + pl.b_off;
        }
        GemmArgs gp{Ap, Bp, C, M, pl.Np, pl.Kp, pl.Kp, transB ? pl.Kp : pl.Np, N, 0, 0, 0, alpha, beta, 0, 0, bias, act, act_param};
        if (pl.Np != N) gp.c_cols = N;
        return transB ? dispatch_gemm<float, float, true>(gp, 1, stream, 0) : dispatch_gemm<float, float, false>(gp, 1, stream, 0);
    }
    int ks32 = 0;
    const int kper32 = (force_tile == 0 && workspace && !transB && batch == 1 && skinny32_applies(M, N, K)) ? 32 * skinny32_plan(N, K, &ks32) : 0;
    if (kper32 && aligned16(A) && aligned16(B) && (size_t)ks32 * M * N * sizeof(float) <= workspace_bytes) {
        const int ks = ks32, kper = kper32;
        constexpr int smem = SKINNY32_STAGES * (32 * 128 + 32 * 512);
        static unsigned long long attr_done = 0;
        if (hipError_t e0 = ensure_dynamic_smem((const void*)gemm_skinny32_kernel<SKINNY32_STAGES>, smem, &attr_done)) return e0;
        hipLaunchKernelGGL(gemm_skinny32_kernel<SKINNY32_STAGES>, dim3((unsigned)(N / 128), (unsigned)ks), dim3(256), smem, stream, g, (float*)workspace, ks, kper);
        if (hipError_t e = hipGetLastError()) return e;
        const long long total = (long long)M * N;
        hipLaunchKernelGGL((skinny_reduce_kernel<float>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, (const float*)workspace,
                           C, M, N, ks, bias, act, act_param, alpha, beta);
        return hipGetLastError();
    }
    if (force_tile == 0 && workspace && batch == 1) {
        // few tiles over a long K: the K ranges run as batches into fp32 partials, summed in range order (deterministic)
        // by the pass that also applies alpha, beta, bias and activation
        const int ks = splitk32_ranges(M, N, K);
        if (ks > 1 && (size_t)ks * M * N * sizeof(float) <= workspace_bytes) {
            GemmArgs gp = g;
            gp.C = workspace; gp.K = K / ks; gp.ldc = N; gp.alpha = 1.0f; gp.beta = 0.0f;
            gp.sA = K / ks; gp.sB = transB ? (long long)(K / ks) : (long long)(K / ks) * N; gp.sC = (long long)M * N;
            gp.bias = nullptr; gp.act = 0;
            hipError_t e = transB ? dispatch_gemm<float, float, true>(gp, ks, stream, 0) : dispatch_gemm<float, float, false>(gp, ks, stream, 0);
            if (e != hipSuccess) return e;
            const long long total = (long long)M * N;
            hipLaunchKernelGGL((skinny_reduce_kernel<float>), dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, (const float*)workspace,
                               C, M, N, ks, bias, act, act_param, alpha, beta);
            return hipGetLastError();
        }
    }
    if (transB) return dispatch_gemm<float, float, true>(g, batch, stream, force_tile);
    return dispatch_gemm<float, float, false>(g, batch, stream, force_tile);
}

// fp32 A [M,K] x fp16 weights B [K,N] -> fp32 C, optional fused epilogue
hipError_t gemm_f32_f16weight(hipStream_t stream, const float* A, const uint16_t* B, float* C, int M, int N, int K,
                              int force_tile, const float* bias, int act, float act_param, void* workspace, size_t workspace_bytes)
{
    GemmArgs g{A, B, C, M, N, K, K, N, N, 0, 0, 0, 1.0f, 0.0f, 0, 0, bias, act, act_param};
    if (force_tile == 0 && workspace && smallm_applies(M, N, K) && gemm_smallm_workspace_bytes(M, N, K) <= workspace_bytes)
        return launch_smallm<true>(g, stream, (float*)workspace);
    // rows of A in 16-byte steps, rows of the fp16 B in 8-byte steps
    const bool vec = aligned16(A) && K % 4 == 0 && (((uintptr_t)B) & 7u) == 0 && N % 4 == 0;
    auto tiles = [&](int bm, int bn) { return (long long)((M + bm - 1) / bm) * ((N + bn - 1) / bn); };
    int tile = force_tile == 64 || force_tile == 128 ? force_tile : choose_tile(tiles(128, 128), tiles(64, 64), 0.85);
    if (tile == 128) {
        if (vec) return launch_gemm<float, float, 128, 128, 2, 2, false, true, true, 1, true>(g, 1, stream);
        return launch_gemm<float, float, 128, 128, 2, 2, false, false, true, 1, true>(g, 1, stream);
    }
    if (vec) return launch_gemm<float, float, 64, 64, 2, 2, false, true, true, 1, true>(g, 1, stream);
    return launch_gemm<float, float, 64, 64, 2, 2, false, false, true, 1, true>(g, 1, stream);
}

#endif

// one 16-bit type per part: T = f16_t in part 1, bf16_t in part 2; out32: C is fp32 (else the same 16-bit type as the inputs)
template <typename T>
static hipError_t gemm_16_typed(hipStream_t stream, const uint16_t* A, const uint16_t* B, void* C, int out32,
                                int M, int N, int K, int force_tile, void* workspace, size_t workspace_bytes, const float* bias, int act,
                                float act_param, const uint16_t* Bpre = nullptr)
{
    // Every plan below that writes to the workspace holds its own need against workspace_bytes first and is passed over when the
    // bytes do not suffice (the tiled kernels at the end need none).
    if (!workspace) workspace_bytes = 0;
    // Bpre: B already packed by gemm_16_pack_b (B itself is then not read); such a call always takes the padded shapes
    PadPlan pl;
    if (Bpre && !(workspace && aligned16(C) && aligned16(workspace) && aligned16(Bpre) && pad16_layout(M, N, K, &pl) && pl.total <= workspace_bytes))
        return hipErrorInvalidValue;
    if (Bpre || (force_tile == 0 && workspace && aligned16(C) && aligned16(workspace) && pad16_plan(M, N, K, &pl) && pl.total <= workspace_bytes)) {
        unsigned char* w = (unsigned char*)workspace;
        const bool padA = pl.Kp != K, padC = pl.Np != N;
        const uint16_t* Ap = A;
        if (padA) {
            if (hipError_t e = pad_rows(stream, A, w + pl.a_off, M, K, M, pl.Kp, 2)) return e;
            Ap = (const uint16_t*)(w + pl.a_off);
        }
        const uint16_t* Bp = Bpre;
        if (!Bpre) {
            if (hipError_t e = pad_rows(stream, B, w + pl.b_off, K, N, pl.Kp, pl.Np, 2)) return e;
            Bp = (const uint16_t*)(w + pl.b_off);
        }
        const float* bp = bias;
        if (bias && padC) {
            if (hipError_t e = pad_rows(stream, bias, w + pl.bias_off, 1, N, 1, pl.Np, 4)) return e;
            bp = (const float*)(w + pl.bias_off);
        }
        if (padC && pl.Np % 128 == 0 && pl.Kp < (1 << 21) && pl.Np < (1 << 21)) {
            // the 16 x 16 x 32 kernel stores the N real columns straight into the caller's C
            GemmArgs gp{Ap, Bp, C, M, pl.Np, pl.Kp, pl.Kp, pl.Np, N, 0, 0, 0, 1.0f, 0.0f, 0, 0, bp, act, act_param};
            gp.c_cols = N;
            const int wd = aligned16(Ap) ? dl16_width(M, pl.Np, pl.Kp, 1) : 0;
            if (wd == 4) return out32 ? launch_gemm_dl16<T, float, 4>(gp, 1, stream) : launch_gemm_dl16<T, T, 4>(gp, 1, stream);
            if (wd == 3) return out32 ? launch_gemm_dl16<T, float, 3>(gp, 1, stream) : launch_gemm_dl16<T, T, 3>(gp, 1, stream);
            if (wd == 2) return out32 ? launch_gemm_dl16<T, float, 2>(gp, 1, stream) : launch_gemm_dl16<T, T, 2>(gp, 1, stream);
            if (wd == 1) return out32 ? launch_gemm_dl16<T, float, 2, true>(gp, 1, stream) : launch_gemm_dl16<T, T, 2, true>(gp, 1, stream);
            if (wd == 5) return out32 ? launch_gemm_dl16<T, float, 2, true, 2>(gp, 1, stream) : launch_gemm_dl16<T, T, 2, true, 2>(gp, 1, stream);
        }
        void* Cp = padC ? (void*)(w + pl.c_off) : C;
        if (hipError_t e = gemm_16_typed<T>(stream, Ap, Bp, Cp, out32, M, pl.Np, pl.Kp, 0,
                                            pl.total > pl.inner_off ? (void*)(w + pl.inner_off) : nullptr,
                                            pl.total > pl.inner_off ? pl.total - pl.inner_off : 0, bp, act, act_param)) return e;
        return padC ? unpad_rows(stream, Cp, C, M, N, pl.Np, out32 ? 4 : 2) : hipSuccess;
    }
    GemmArgs g{A, B, C, M, N, K, K, N, N, 0, 0, 0, 1.0f, 0.0f, 0, 0, bias, act, act_param};
    if (force_tile == 0 && workspace && skinny_applies(M, N, K) && aligned16(A) && aligned16(B) &&
        (size_t)skinny_ksplit(N, K) * M * N * sizeof(float) <= workspace_bytes) {
        float* ws = (float*)workspace;
        return out32 ? launch_skinny<T, float>(g, stream, ws) : launch_skinny<T, T>(g, stream, ws);
    }
    if (force_tile == 0 && dl16_applies<float>(g)) {
        if (const int first = msplit16_rows(M, N, K)) {
            // the rows of the whole rounds, then the rest (stream order; the two share the workspace one after the other)
            if (hipError_t e = gemm_16_typed<T>(stream, A, B, C, out32, first, N, K, 0, workspace, workspace_bytes, bias, act, act_param)) return e;
            return gemm_16_typed<T>(stream, A + (size_t)first * K, B, (unsigned char*)C + (size_t)first * N * (out32 ? 4 : 2), out32, M - first, N, K, 0,
                                    workspace, workspace_bytes, bias, act, act_param);
        }
    }
    if (force_tile == 0 && workspace) {
        int big = 0;
        const int ks = splitk16_ranges(M, N, K, &big);
        if (ks && (size_t)ks * M * N * sizeof(float) <= workspace_bytes) {
            GemmArgs gp = g;
            gp.C = workspace; gp.K = K / ks; gp.ldc = N;
            gp.sA = K / ks; gp.sB = (long long)(K / ks) * N; gp.sC = (long long)M * N;
            gp.bias = nullptr; gp.act = 0;
            if (dl16_applies<float>(gp)) {
                if (hipError_t e = big ? launch_gemm_dl16<T, float, 4>(gp, ks, stream) : launch_gemm_dl16<T, float, 2, true>(gp, ks, stream)) return e;
                const long long total = (long long)M * N;
                const unsigned grid = (unsigned)((total + 255) / 256);
                if (out32) hipLaunchKernelGGL((skinny_reduce_kernel<float>), dim3(grid), dim3(256), 0, stream, (const float*)workspace, C, M, N, ks, bias, act, act_param, 1.0f, 0.0f);
                else hipLaunchKernelGGL((skinny_reduce_kernel<T>), dim3(grid), dim3(256), 0, stream, (const float*)workspace, C, M, N, ks, bias, act, act_param, 1.0f, 0.0f);
                return hipGetLastError();
            }
        }
    }
    if (out32) return dispatch_gemm<T, float, false>(g, 1, stream, force_tile);
    return dispatch_gemm<T, T, false>(g, 1, stream, force_tile);
}

hipError_t gemm_16_f16(hipStream_t stream, const uint16_t* A, const uint16_t* B, void* C, int out32,
                       int M, int N, int K, int force_tile, void* workspace, size_t workspace_bytes, const float* bias, int act, float act_param, const uint16_t* Bpre);
hipError_t gemm_16_bf16(hipStream_t stream, const uint16_t* A, const uint16_t* B, void* C, int out32,
                        int M, int N, int K, int force_tile, void* workspace, size_t workspace_bytes, const float* bias, int act, float act_param, const uint16_t* Bpre);
hipError_t gemm_16_rope_f16(hipStream_t stream, const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K, int force_tile,
                            void* workspace, size_t workspace_bytes, const RopeEpilogue& rope);
hipError_t gemm_16_rope_bf16(hipStream_t stream, const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K, int force_tile,
                             void* workspace, size_t workspace_bytes, const RopeEpilogue& rope);
// C = A B, then interleaved RoPE over the leading columns of C (launch.hpp)
template <typename T>
static hipError_t gemm_16_rope_typed(hipStream_t stream, const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K, int force_tile,
                                     void* workspace, size_t workspace_bytes, const RopeEpilogue& rope)
{
    if (!workspace) workspace_bytes = 0;
    // the plan of gemm_16_typed that sums K ranges in a pass of its own takes the rotation into that pass
    if (force_tile == 0 && workspace && skinny_applies(M, N, K) && aligned16(A) && aligned16(B) &&
        (size_t)skinny_ksplit(N, K) * M * N * sizeof(float) <= workspace_bytes) {
        GemmArgs g{A, B, C, M, N, K, K, N, N, 0, 0, 0, 1.0f, 0.0f, 0, 0, nullptr, 0, 0.0f};
        return launch_skinny<T, T>(g, stream, (float*)workspace, &rope);
    }
    if (hipError_t e = gemm_16_typed<T>(stream, A, B, C, 0, M, N, K, force_tile, workspace, workspace_bytes, nullptr, 0, 0.0f)) return e;
    return rope_cols16(stream, std::is_same<T, f16_t>::value ? 1 : 2, C, rope.cosc, rope.sinc, M, N, rope.cols, rope.head_dim, rope.seq_len, rope.start_position);
}

#if AIDN_GEMM_PART == 1
hipError_t gemm_16_f16(hipStream_t stream, const uint16_t* A, const uint16_t* B, void* C, int out32,
                       int M, int N, int K, int force_tile, void* workspace, size_t workspace_bytes, const float* bias, int act, float act_param, const uint16_t* Bpre)
{ return gemm_16_typed<f16_t>(stream, A, B, C, out32, M, N, K, force_tile, workspace, workspace_bytes, bias, act, act_param, Bpre); }
hipError_t gemm_16_rope_f16(hipStream_t stream, const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K, int force_tile,
                            void* workspace, size_t workspace_bytes, const RopeEpilogue& rope)
{ return gemm_16_rope_typed<f16_t>(stream, A, B, C, M, N, K, force_tile, workspace, workspace_bytes, rope); }
#elif AIDN_GEMM_PART == 2
hipError_t gemm_16_bf16(hipStream_t stream, const uint16_t* A, const uint16_t* B, void* C, int out32,
                        int M, int N, int K, int force_tile, void* workspace, size_t workspace_bytes, const float* bias, int act, float act_param, const uint16_t* Bpre)
{ return gemm_16_typed<bf16_t>(stream, A, B, C, out32, M, N, K, force_tile, workspace, workspace_bytes, bias, act, act_param, Bpre); }
hipError_t gemm_16_rope_bf16(hipStream_t stream, const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K, int force_tile,
                             void* workspace, size_t workspace_bytes, const RopeEpilogue& rope)
{ return gemm_16_rope_typed<bf16_t>(stream, A, B, C, M, N, K, force_tile, workspace, workspace_bytes, rope); }
#else
// kind: 0 = fp16, 1 = bf16
hipError_t gemm_16(hipStream_t stream, int kind, const uint16_t* A, const uint16_t* B, void* C, int out32,
                   int M, int N, int K, int force_tile, void* workspace, size_t workspace_bytes, const float* bias, int act, float act_param, const uint16_t* Bpre)
{
    if (kind == 0) return gemm_16_f16(stream, A, B, C, out32, M, N, K, force_tile, workspace, workspace_bytes, bias, act, act_param, Bpre);
    return gemm_16_bf16(stream, A, B, C, out32, M, N, K, force_tile, workspace, workspace_bytes, bias, act, act_param, Bpre);
}
hipError_t gemm_16_rope(hipStream_t stream, int kind, const uint16_t* A, const uint16_t* B, uint16_t* C, int M, int N, int K, int force_tile,
                        void* workspace, size_t workspace_bytes, const RopeEpilogue& rope)
{
    if (kind == 0) return gemm_16_rope_f16(stream, A, B, C, M, N, K, force_tile, workspace, workspace_bytes, rope);
    return gemm_16_rope_bf16(stream, A, B, C, M, N, K, force_tile, workspace, workspace_bytes, rope);
}
#endif

}  // namespace aidn
