// Decode attention (one query row per (batch, head)) for gfx950.  HBM-bound: each K and V row is
// read exactly once with 128-bit loads, LPK lanes per row so one wave load covers 64/LPK whole
// consecutive rows (1 KiB contiguous when the cache is dense); no MFMA.
//
// Replaces FlashDecode (src/AiDotNet.Tensors/Engines/DirectGpu/HIP/HipBackend.cs:919-965, kernel
// strings Kernels/HipFlashDecodeKernels.cs:21-83: one THREAD per (head, split)) and the Sq == 1 use
// of ScaledDotProductAttention (Kernels/HipAttentionKernels.cs:33-125).  Value semantics: the
// reference decode test's oracle (tests/AiDotNet.Tensors.Tests/Engines/DirectGpu/
// FlashDecodeHipTests.cs:43-69), i.e. softmax(scale * q.K^T) V over all cached keys.
//
// grid = (B*H / heads per workgroup) * splits, 256 threads.  Wave w of the workgroup walks its split in blocks of
// U * KPW keys (KPW = 64 / LPK keys per load, U loads in flight for K and U for V).  Every lane
// keeps an online-softmax state (m, l, acc[E]) for its key slot and its 16-byte slice of the head
// dim; slots and waves are merged through LDS, splits through a workspace and a second kernel.
#include "common.hpp"
#include "launch.hpp"

namespace aidn {

struct DecodeArgs {
    const void* q; const void* k; const void* v; void* o; float* lse;
    float* ws;               // [B*H][splits][2 + DPAD] : m, l, acc[DPAD]   (splits > 1)
    int B, H, Hkv, Sk, D;
    float scale;
    int splits, chunk;       // keys per split
    long long qs[2], ks[3], vs[3], os[2];   // q/o: batch, head; k/v: batch, head, row
    int vec_in;
    const int* bt; int bsz; long long bt_bs;   // block table of a paged cache (null = contiguous), block size, batch stride
};

template <typename T> struct Raw3;
template <> struct Raw3<float> { typedef uint32_t type; };
template <> struct Raw3<f16_t> { typedef uint16_t type; };
template <> struct Raw3<bf16_t> { typedef uint16_t type; };

// STREAM: a row of the K/V cache, read once per launch: a non-temporal load (a plain read loop reaches 6.0-6.2 TB/s on this part,
// the same loop with non-temporal loads 6.9-7.0 TB/s)
template <typename T, bool STREAM = false>
__device__ __forceinline__ u32x4 ld16d(const typename Raw3<T>::type* p, int valid, bool vec)
{
    u32x4 v = {0u, 0u, 0u, 0u};
    if (valid <= 0) return v;
    if (vec && valid >= Elem<T>::PER16) return STREAM ? __builtin_nontemporal_load((const u32x4*)p) : *(const u32x4*)p;
    if constexpr (Elem<T>::BYTES == 4) {
#pragma unroll
        for (int e = 0; e < 4; e++) if (e < valid) v[e] = p[e];
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) if (e < valid) v[e >> 1] |= ((uint32_t)p[e]) << (16 * (e & 1));
    }
    return v;
}

// widen one 16-byte fragment to E floats
template <typename T>
__device__ __forceinline__ void widen16(const u32x4& x, float (&f)[Elem<T>::PER16])
{
    if constexpr (Elem<T>::BYTES == 4) {
#pragma unroll
        for (int e = 0; e < 4; e++) f[e] = as_f32(x[e]);
    } else {
#pragma unroll
        for (int w = 0; w < 4; w++) {
            f[2 * w] = Elem<T>::widen(x[w] & 0xFFFFu);
            f[2 * w + 1] = Elem<T>::widen(x[w] >> 16);
        }
    }
}

// Sum over the LPK consecutive lanes that share a key row (LPK a power of two >= 4, aligned): quad permutes and row mirrors are
// VALU data-parallel-primitive operands (no LDS round trip); beyond a 16-lane row one permute and the half-wave swap.
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v)
{
    return as_f32((uint32_t)__builtin_amdgcn_update_dpp(0, (int)as_u32(v), CTRL, 0xF, 0xF, false));
}
template <int LPK>
__device__ __forceinline__ float group_sum(float p)
{
    p += dpp_f<0xB1>(p);                       // quad_perm [1,0,3,2]
    p += dpp_f<0x4E>(p);                       // quad_perm [2,3,0,1]
    if constexpr (LPK >= 8) p += dpp_f<0x141>(p);      // row_half_mirror
    if constexpr (LPK >= 16) p += dpp_f<0x140>(p);     // row_mirror
    if constexpr (LPK >= 32) p += shfl_xor_f(p, 16);
    if constexpr (LPK >= 64) p = sum_with_partner32(p);
    return p;
}

constexpr float D_LOG2E = 1.4426950408889634f;
constexpr float D_LN2 = 0.6931471805599453f;

// GH: query heads of one K/V head that a workgroup serves from the same loads (1 = one head per workgroup).  The K/V rows of a
// grouped-query cache are then fetched once per GH query heads instead of once per head.
template <typename T, typename OutT, int LPK, int U, int GH>
__global__ __launch_bounds__(256) void decode_partial_kernel(const DecodeArgs a)
{
    typedef typename Raw3<T>::type raw_t;
    constexpr int E = Elem<T>::PER16;
    constexpr int KPW = 64 / LPK;          // keys per wave load
    constexpr int NWV = 4;
    constexpr int DPAD = LPK * E;          // padded head dim
    constexpr int SLOTS = NWV * KPW;

    __shared__ float s_m[SLOTS], s_l[SLOTS];
    __shared__ float s_acc[SLOTS][DPAD + 4];

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int dl = lane % LPK, sk = lane / LPK;
    // one grid dimension (y and z are limited to 65535): the splits of a (batch, K/V head, chunk of GH query heads) are neighbours
    const int split = blockIdx.x % a.splits;
    const int gq = a.H / a.Hkv;                    // query heads per K/V head (a multiple of GH)
    const int chunks = gq / GH;
    const int by = blockIdx.x / a.splits;
    const int b = by / (a.Hkv * chunks);
    const int kvh = (by - b * a.Hkv * chunks) / chunks;
    const int hd0 = kvh * gq + (by % chunks) * GH;  // first query head
    const bool vec = a.vec_in != 0;
    const int d0 = dl * E;

    const raw_t* __restrict__ K = (const raw_t*)a.k + b * a.ks[0] + kvh * a.ks[1];
    const raw_t* __restrict__ V = (const raw_t*)a.v + b * a.vs[0] + kvh * a.vs[1];
    const int* __restrict__ bt = a.bt ? a.bt + b * a.bt_bs : nullptr;

    float qf[GH][E];
#pragma unroll
    for (int g = 0; g < GH; g++) {
        const raw_t* __restrict__ Q = (const raw_t*)a.q + b * a.qs[0] + (hd0 + g) * a.qs[1];
        u32x4 qx = ld16d<T>(Q + d0, a.D - d0, vec);
        widen16<T>(qx, qf[g]);
        const float sl2 = a.scale * D_LOG2E;
#pragma unroll
        for (int e = 0; e < E; e++) qf[g][e] *= sl2;      // scores come out in the log2 domain
    }

    const int kbeg = split * a.chunk;
    const int kend = min(a.Sk, kbeg + a.chunk);

    float m_run[GH], l_run[GH];
    float acc[GH][E];
#pragma unroll
    for (int g = 0; g < GH; g++) {
        m_run[g] = -INFINITY; l_run[g] = 0.0f;
#pragma unroll
        for (int e = 0; e < E; e++) acc[g][e] = 0.0f;
    }

    for (int base = kbeg + wave * (U * KPW); base < kend; base += NWV * U * KPW) {
        u32x4 kx[U], vx[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            int key = base + u * KPW + sk;
            bool ok = key < kend;
            const long long row = ok ? paged_row(bt, a.bsz, key) : 0;
            kx[u] = ok ? ld16d<T, true>(K + row * a.ks[2] + d0, a.D - d0, vec) : u32x4{0u, 0u, 0u, 0u};
            vx[u] = ok ? ld16d<T, true>(V + row * a.vs[2] + d0, a.D - d0, vec) : u32x4{0u, 0u, 0u, 0u};
        }
        float s[GH][U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            float kf[E];
            widen16<T>(kx[u], kf);
            const bool live = base + u * KPW + sk < kend;
#pragma unroll
            for (int g = 0; g < GH; g++) {
                float p = 0.0f;
#pragma unroll
                for (int e = 0; e < E; e++) p = fmaf(qf[g][e], kf[e], p);
                p = group_sum<LPK>(p);
                s[g][u] = live ? p : -INFINITY;
            }
        }
        float pr[GH][U];
#pragma unroll
        for (int g = 0; g < GH; g++) {
            float mloc = s[g][0];
#pragma unroll
            for (int u = 1; u < U; u++) mloc = fmaxf(mloc, s[g][u]);
            const float m_new = fmaxf(m_run[g], mloc);
            const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m_run[g] - m_use);
            m_run[g] = m_new;
            float l = l_run[g] * alpha;
#pragma unroll
            for (int e = 0; e < E; e++) acc[g][e] *= alpha;
#pragma unroll
            for (int u = 0; u < U; u++) {
                pr[g][u] = __builtin_amdgcn_exp2f(s[g][u] - m_use);
                l += pr[g][u];
            }
            l_run[g] = l;
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            float vf[E];
            widen16<T>(vx[u], vf);
#pragma unroll
            for (int g = 0; g < GH; g++)
#pragma unroll
                for (int e = 0; e < E; e++) acc[g][e] = fmaf(pr[g][u], vf[e], acc[g][e]);
        }
    }

    // ---- merge the key slots of all waves, one query head at a time through the same LDS
    const int slot = wave * KPW + sk;
#pragma unroll
    for (int g = 0; g < GH; g++) {
        if (g > 0) __syncthreads();
        if (dl == 0) { s_m[slot] = m_run[g]; s_l[slot] = l_run[g]; }
#pragma unroll
        for (int e = 0; e < E; e++) s_acc[slot][d0 + e] = acc[g][e];
        __syncthreads();

        const int hd = hd0 + g;
        const int bh = b * a.H + hd;
        float M = -INFINITY;
#pragma unroll
        for (int i = 0; i < SLOTS; i++) M = fmaxf(M, s_m[i]);
        const float Muse = (M == -INFINITY) ? 0.0f : M;
        for (int d = t; d < DPAD; d += 256) {
            float L = 0.0f, A = 0.0f;
#pragma unroll
            for (int i = 0; i < SLOTS; i++) {
                float w = __builtin_amdgcn_exp2f(s_m[i] - Muse);
                L += s_l[i] * w;
                A += s_acc[i][d] * w;
            }
            if (a.splits > 1) {
                float* ws = a.ws + ((long long)bh * a.splits + split) * (2 + DPAD);
                if (d == 0) { ws[0] = M; ws[1] = L; }
                ws[2 + d] = A;
            } else if (d < a.D) {
                typedef typename Raw3<OutT>::type out_t;
                out_t* O = (out_t*)a.o + b * a.os[0] + hd * a.os[1];
                float r = L > 0.0f ? A / L : 0.0f;
                if constexpr (Elem<OutT>::BYTES == 4) O[d] = as_u32(r);
                else O[d] = (out_t)Elem<OutT>::narrow(r);
                if (d == 0 && a.lse) a.lse[bh] = L > 0.0f ? (M + __builtin_amdgcn_logf(L)) * D_LN2 : -INFINITY;
            }
        }
    }
}

// Merge the per-split (m, l, acc) triples: grid = B*H, one thread per head-dim element.  The split weights are formed once per
// head (through LDS); the partial rows are then read eight splits at a time so that the loads of a thread overlap.
template <typename OutT>
__global__ __launch_bounds__(256) void decode_reduce_kernel(const DecodeArgs a, int dpad)
{
    __shared__ float s_w[64], s_ml[2];
    const int bh = blockIdx.x;
    const int b = bh / a.H, hd = bh - b * a.H;
    const long long stride = 2 + dpad;
    const float* ws = a.ws + (long long)bh * a.splits * stride;
    const int t = threadIdx.x;
    // splits <= 64: lane s of the first wave holds split s
    if (t < 64) {
        const float m = t < a.splits ? ws[t * stride] : -INFINITY;
        const float l = t < a.splits ? ws[t * stride + 1] : 0.0f;
        float M = m;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) M = fmaxf(M, shfl_xor_f(M, off));
        const float Muse = (M == -INFINITY) ? 0.0f : M;
        const float w = __builtin_amdgcn_exp2f(m - Muse);
        float L = l * w;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) L += shfl_xor_f(L, off);
        s_w[t] = w;
        if (t == 0) { s_ml[0] = M; s_ml[1] = L; }
    }
    __syncthreads();
    const float M = s_ml[0], L = s_ml[1];
    for (int d = t; d < a.D; d += blockDim.x) {
        float A = 0.0f;
        int s0 = 0;
        for (; s0 + 8 <= a.splits; s0 += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = ws[(s0 + u) * stride + 2 + d];
#pragma unroll
            for (int u = 0; u < 8; u++) A += v[u] * s_w[s0 + u];
        }
        for (; s0 < a.splits; s0++) A += ws[s0 * stride + 2 + d] * s_w[s0];
        typedef typename Raw3<OutT>::type out_t;
        out_t* O = (out_t*)a.o + b * a.os[0] + hd * a.os[1];
        float r = L > 0.0f ? A / L : 0.0f;
        if constexpr (Elem<OutT>::BYTES == 4) O[d] = as_u32(r);
        else O[d] = (out_t)Elem<OutT>::narrow(r);
        if (d == 0 && a.lse) a.lse[bh] = L > 0.0f ? (M + __builtin_amdgcn_logf(L)) * D_LN2 : -INFINITY;
    }
}

// ------------------------------------------------------------------ host side
static int lanes_per_key(int D, int eb)
{
    int chunks = (D * eb + 15) / 16;
    int lpk = 1;
    while (lpk < chunks) lpk <<= 1;
    return lpk;
}

static int effective_sk(const AttnParams& p)
{
    // Sq == 1: key j is masked iff j > 0 + qoff
    if (!p.causal) return p.Sk;
    long long lim = (long long)p.qoff + 1;
    if (lim < 0) lim = 0;
    return (int)(lim < p.Sk ? lim : p.Sk);
}

int attn_decode_splits(int kind, const AttnParams& p, int splits)
{
    const int sk = effective_sk(p);
    int maxs = (sk + 255) / 256;            // at least 256 keys per split
    if (maxs < 1) maxs = 1;
    if (splits <= 0) {
        // workgroups per split: one per query head, or one per K/V head when the grouped form runs
        const int gq = p.Hkv > 0 ? p.H / p.Hkv : 1;
        const bool grouped = attn_group_decode_applies(kind, p);
        long long bh = (long long)p.B * (grouped ? p.Hkv : p.H / (gq % 4 == 0 ? 4 : gq % 2 == 0 ? 2 : 1));
        // about four workgroups per CU for the per-head kernel, rounded to the nearest count (a grid that is already that large is not
        // split: the merge pass costs more than it balances); the grouped form (one computing wave per workgroup, a key tile per
        // barrier) is fastest at about two per CU (B32 H32 Hkv8 KV4096: 85 us with 2 ranges, 92 with 8; B8 KV8192: 46 with 8, 54 with 32)
        splits = grouped ? (int)((512 + bh - 1) / bh) : (int)((1024 + bh / 2) / bh);
    }
    if (splits > maxs) splits = maxs;
    if (splits > 64) splits = 64;
    if (splits < 1) splits = 1;
    return splits;
}

size_t attn_decode_workspace_bytes(const AttnParams& p, int eff_splits)
{
    if (eff_splits <= 1) return 0;
    // padded head dim of whichever element size is used: take the larger of the two
    int l4 = lanes_per_key(p.D, 4), l2 = lanes_per_key(p.D, 2);
    if (l4 < 4) l4 = 4;
    if (l2 < 4) l2 = 4;
    int dpad = l4 * 4 > l2 * 8 ? l4 * 4 : l2 * 8;
    return (size_t)p.B * p.H * eff_splits * (2 + dpad) * sizeof(float);
}

template <typename T, typename OutT, int LPK, int U>
static hipError_t launch_decode(DecodeArgs a, hipStream_t stream)
{
    constexpr int DPAD = LPK * Elem<T>::PER16;
    // query heads of a K/V head that share a workgroup (and its loads): 4, 2 or 1, whichever divides the group
    const int gq = a.H / a.Hkv;
    const int gh = gq % 4 == 0 ? 4 : gq % 2 == 0 ? 2 : 1;
    const long long nwg = (long long)a.B * a.H / gh * a.splits;
    if (nwg > 0x7FFFFFFFLL) return hipErrorInvalidValue;
    dim3 grid((unsigned)nwg);
    if (gh == 4) hipLaunchKernelGGL((decode_partial_kernel<T, OutT, LPK, U, 4>), grid, dim3(256), 0, stream, a);
    else if (gh == 2) hipLaunchKernelGGL((decode_partial_kernel<T, OutT, LPK, U, 2>), grid, dim3(256), 0, stream, a);
    else hipLaunchKernelGGL((decode_partial_kernel<T, OutT, LPK, U, 1>), grid, dim3(256), 0, stream, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (a.splits > 1) {
        int threads = a.D <= 64 ? 64 : (a.D <= 128 ? 128 : 256);
        hipLaunchKernelGGL((decode_reduce_kernel<OutT>), dim3((unsigned)(a.B * a.H)), dim3(threads), 0, stream, a, DPAD);
        e = hipGetLastError();
    }
    return e;
}

template <typename T, typename OutT>
static hipError_t dispatch_decode(const DecodeArgs& a, hipStream_t stream)
{
    const int lpk = lanes_per_key(a.D, Elem<T>::BYTES);
    switch (lpk) {
    case 1: case 2: case 4: return launch_decode<T, OutT, 4, 4>(a, stream);
    case 8: return launch_decode<T, OutT, 8, 4>(a, stream);
    case 16: return launch_decode<T, OutT, 16, 4>(a, stream);
    case 32: return launch_decode<T, OutT, 32, 4>(a, stream);
    case 64: return launch_decode<T, OutT, 64, 4>(a, stream);
    default: return hipErrorInvalidValue;
    }
}

hipError_t attn_decode(hipStream_t stream, int kind, const AttnParams& p, int eff_splits, void* workspace)
{
    if (attn_group_decode_applies(kind, p) && effective_sk(p) > 0) {
        const int sk = effective_sk(p);
        int chunk = (sk + eff_splits - 1) / eff_splits;
        chunk = (chunk + 63) / 64 * 64;
        if (hipError_t e = attn_group_decode(stream, kind, p, sk, eff_splits, chunk, (float*)workspace)) return e;
        if (eff_splits > 1) {
            DecodeArgs r;
            r.q = nullptr; r.k = nullptr; r.v = nullptr; r.o = p.o; r.lse = p.lse; r.ws = (float*)workspace;
            r.B = p.B; r.H = p.H; r.Hkv = p.Hkv; r.Sk = sk; r.D = p.D; r.scale = p.scale; r.splits = eff_splits; r.chunk = chunk;
            r.qs[0] = p.qs[0]; r.qs[1] = p.qs[1]; r.os[0] = p.os[0]; r.os[1] = p.os[1];
            for (int i = 0; i < 3; i++) { r.ks[i] = p.ks[i]; r.vs[i] = p.vs[i]; }
            r.vec_in = 1; r.bt = nullptr; r.bsz = 0; r.bt_bs = 0;
            const dim3 grid((unsigned)(p.B * p.H));
            if (!p.out16) hipLaunchKernelGGL((decode_reduce_kernel<float>), grid, dim3(128), 0, stream, r, 128);
            else if (kind == 1) hipLaunchKernelGGL((decode_reduce_kernel<f16_t>), grid, dim3(128), 0, stream, r, 128);
            else hipLaunchKernelGGL((decode_reduce_kernel<bf16_t>), grid, dim3(128), 0, stream, r, 128);
            return hipGetLastError();
        }
        return hipSuccess;
    }
    DecodeArgs a;
    a.q = p.q; a.k = p.k; a.v = p.v; a.o = p.o; a.lse = p.lse; a.ws = (float*)workspace;
    a.B = p.B; a.H = p.H; a.Hkv = p.Hkv; a.Sk = effective_sk(p); a.D = p.D;
    a.scale = p.scale;
    a.splits = eff_splits;
    a.qs[0] = p.qs[0]; a.qs[1] = p.qs[1]; a.os[0] = p.os[0]; a.os[1] = p.os[1];
    for (int i = 0; i < 3; i++) { a.ks[i] = p.ks[i]; a.vs[i] = p.vs[i]; }
    a.bt = p.block_table; a.bsz = p.block_size; a.bt_bs = p.block_table_stride;
    const int eb = kind == 0 ? 4 : 2, e = 16 / eb;
    const int lpk = lanes_per_key(p.D, eb) < 4 ? 4 : lanes_per_key(p.D, eb);
    // keys per split: a multiple of the keys one workgroup iteration covers
    const int step = 4 * 4 * (64 / lpk);
    int chunk = (a.Sk + eff_splits - 1) / eff_splits;
    chunk = ((chunk + step - 1) / step) * step;
    if (chunk < step) chunk = step;
    a.chunk = chunk;
    auto al = [](const void* ptr, const long long* s, int n, int bytes) {
        bool ok = ((uintptr_t)ptr & 15u) == 0;
        for (int i = 0; i < n; i++) ok = ok && (s[i] * bytes) % 16 == 0;
        return ok;
    };
    a.vec_in = (p.D % e == 0) && al(p.q, p.qs, 2, eb) && al(p.k, p.ks, 3, eb) && al(p.v, p.vs, 3, eb);
    if (kind == 0) return dispatch_decode<float, float>(a, stream);
    if (kind == 1) return p.out16 ? dispatch_decode<f16_t, f16_t>(a, stream) : dispatch_decode<f16_t, float>(a, stream);
    return p.out16 ? dispatch_decode<bf16_t, bf16_t>(a, stream) : dispatch_decode<bf16_t, float>(a, stream);
}

}  // namespace aidn
