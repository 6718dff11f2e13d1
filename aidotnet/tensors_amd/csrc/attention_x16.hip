// Fused attention forward for the 16-bit types at head dimension 128 (plain or causal, aligned contiguous K/V) on
// v_mfma_f32_16x16x32_{f16,bf16}: the prefill form of FlashAttentionV2 / ScaledDotProductAttention behind the reference's
// backend slot (src/AiDotNet.Tensors/Engines/DirectGpu/HIP/HipBackend.cs:6118-6302; value semantics
// src/AiDotNet.Tensors/Engines/CpuEngine.cs:29146-29288, update order Engines/Simd/FusedAttention.cs:159-286).
//
// Workgroup: 128 query rows of one (batch, head), four waves of 32 rows (two 16-row blocks qb); K and V stream through LDS
// as 64-key tiles (direct global -> LDS loads, two stages each, one barrier per tile) and are consumed in units of 32 keys.
//   S^T = K Q^T      MFMA rows = keys (16-key block kb), cols = queries: lane (l16, g) holds query l16 of block qb and keys
//                    16 kb + 4 g + 0..3.  Q is held in registers, multiplied once by scale * log2(e) and rounded back to the
//                    storage type; the accumulator of a block starts at -m (the row's exponent reference) instead of zero, so
//                    the MFMA result is already the argument of exp2: no multiply-add per logit.
//   O^T += V^T P^T   MFMA rows = head dimension (16-wide block db), cols = queries.  The B operand of a 32-key step wants
//                    8 k-values per lane: the packed probabilities of blocks kb = 0, 1 in accumulator order, no shuffles.
//                    The k index of that step is thereby a permutation of the keys, k = 8 g + e <-> key 16 (e / 4) + 4 g + e % 4,
//                    which the transposing LDS reads of V^T follow by their row addresses.
// Softmax without a running-maximum pass: the reference m of a row only has to keep exp2 in range, it need not be the
// maximum (LSE = m + log2(l) holds for any m).  It is set from the true row maximum of the first unit and then stands; the
// probabilities of a unit are formed against it at once, and the unit's sum tells whether one of them left the range (only
// then, or in the units at the edges of a wave's key range, the row maxima are formed and O, l and m moved).  Per logit
// that leaves one v_exp_f32, half a packed convert and half a v_dot2 for the row sum.
// Schedule: unit u's exponentials run beside the matrix work of its neighbours -- P(u-1) V and S(u+1) -- so the vector and
// matrix instructions of one iteration are independent streams; LDS fragment reads run three fragments ahead of their MFMAs.
#include "attention_common.hpp"

namespace aidn {

typedef float f32x4a __attribute__((ext_vector_type(4)));

template <typename T> struct MmaX16;
template <> struct MmaX16<f16_t> {
    static __device__ __forceinline__ f32x4a run(const u32x4& a, const u32x4& b, const f32x4a& c)
    { return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0); }
};
template <> struct MmaX16<bf16_t> {
    static __device__ __forceinline__ f32x4a run(const u32x4& a, const u32x4& b, const f32x4a& c)
    { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0); }
};

// 8 stored elements times c, rounded back to the storage type
template <typename T> __device__ __forceinline__ u32x4 scale_frag(const u32x4& f, float c);
template <> __device__ __forceinline__ u32x4 scale_frag<f16_t>(const u32x4& f, float c)
{
    u32x4 r;
#pragma unroll
    for (int w = 0; w < 4; w++) {
        const uint32_t x = f[w];
        r[w] = pack2_p<f16_t>(f16_bits_to_float(x & 0xFFFFu) * c, f16_bits_to_float(x >> 16) * c);
    }
    return r;
}
template <> __device__ __forceinline__ u32x4 scale_frag<bf16_t>(const u32x4& f, float c)
{
    u32x4 r;
#pragma unroll
    for (int w = 0; w < 4; w++) {
        const uint32_t x = f[w];
        r[w] = pack2_p<bf16_t>(as_f32(x << 16) * c, as_f32(x & 0xFFFF0000u) * c);
    }
    return r;
}

#define X16_HEAD_GROUP 4

template <typename T, typename OutT>
__global__ __launch_bounds__(256, 2) void attn_fwd_x16_kernel(const AttnArgs a)
{
    typedef uint16_t raw_t;
    constexpr int BC = 64, BR = 128;
    constexpr int KBYTES = BC * 256, VBYTES = BC * 256;
    constexpr float BIG = 1.152921504606847e18f;       // 2^60: a unit's probability sum beyond it means exp2 left the range

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int l16 = lane & 15, g = lane >> 4;
    int bh, qt;
    {
        int nblk = gridDim.x, pid = blockIdx.x;
        int per = nblk >> 3, rem = nblk & 7;
        int xcd = pid & 7, idx = pid >> 3;
        int logical = (xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per) + idx;
        bh = logical / a.qtiles;
        qt = a.qtiles - 1 - (logical - bh * a.qtiles);
        if (a.paired) {
            // XCD-contiguous heads, qtiles / 2 workgroups per head: first the late (heavy) tile of the pair, then the early one
            const int units = a.qtiles >> 1;
            bh = logical / units;
            qt = a.qtiles - 1 - (logical - bh * units);
        } else if (a.causal) {
            // heads in groups of X16_HEAD_GROUP (their K and V are what an XCD's L2 holds); a group's query tiles heaviest first
            const bool whole = rem == 0 && per % a.qtiles == 0;
            const int heads = whole ? per / a.qtiles : nblk / a.qtiles;
            const int at = whole ? idx : logical;
            const int gsz = heads < X16_HEAD_GROUP ? heads : X16_HEAD_GROUP;
            const int per_group = gsz * a.qtiles;
            const int grp = at / per_group, in = at - grp * per_group;
            const int first = grp * gsz;
            const int cur = heads - first < gsz ? heads - first : gsz;
            qt = a.qtiles - 1 - in / cur;
            bh = (whole ? xcd * heads : 0) + first + in % cur;
        }
    }

    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)smem);
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    const float sl2 = a.scale * LOG2E;
    const int Sk = a.Sk;
    const long long qoff = a.qoff;

    // Direct-to-LDS loads.  This wave's share of a tile: K wave-loads 4 w .. 4 w + 3 and the same of V, each 4 keys x 256 B;
    // lane -> (key = 4 * load + lane / 16, chunk position lane % 16).  LDS layout ([key][256 B], 16-byte chunk c of key k):
    //   K: position c ^ (k & 15)                                   (b128 fragment reads: 16 lanes = 16 keys, one chunk column)
    //   V: position c ^ ((k & 3) << 2) ^ (((k >> 2) & 1) << 1)     (transposing reads: the 8 keys two 16-lane groups touch in one
    //                                                              cycle land in 8 different 32-byte bank groups)
    const int ld_key = lane >> 4, ld_pos = lane & 15;
    const long long k_row_bytes = a.ks[2] * 2, v_row_bytes = a.vs[2] * 2;
    uint32_t k_lane_off[4], v_lane_off[2];
#pragma unroll
    for (int i = 0; i < 4; i++) k_lane_off[i] = (uint32_t)(ld_key * k_row_bytes) + ((ld_pos ^ (4 * i + ld_key)) << 4);
#pragma unroll
    for (int i = 0; i < 2; i++) v_lane_off[i] = (uint32_t)(ld_key * v_row_bytes) + ((ld_pos ^ ((ld_key << 2) ^ (i << 1))) << 4);

    const int npass = a.paired ? 2 : 1;
    for (int pass = 0; pass < npass; pass++) {
    if (pass == 1) qt = a.qtiles - 1 - qt;
    const int b = bh / a.H, hd = bh - b * a.H;
    const int kvh = hd / (a.H / a.Hkv);
    const int q0 = qt * BR;
    const raw_t* __restrict__ Q = (const raw_t*)a.q + b * a.qs[0] + hd * a.qs[1];
    const raw_t* __restrict__ K = (const raw_t*)a.k + b * a.ks[0] + kvh * a.ks[1];
    const raw_t* __restrict__ V = (const raw_t*)a.v + b * a.vs[0] + kvh * a.vs[1];

    auto issue_k = [&](int tile) {
        const uint32_t dst = lds0 + (tile & 1) * KBYTES + wave_s * 4096;
        if (tile * BC + BC <= Sk) {
            const unsigned char* src = (const unsigned char*)K + (long long)(tile * BC + 16 * wave_s) * k_row_bytes;
#pragma unroll
            for (int i = 0; i < 4; i++) attn_dma16_base(src + 4 * i * k_row_bytes, k_lane_off[i], dst + i * 1024);
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int key = 4 * (wave * 4 + i) + ld_key;            // key inside the tile
                const int gkey = min(tile * BC + key, Sk - 1);          // rows past the end are clamped loads, masked later
                attn_dma16(K + (long long)gkey * a.ks[2] + (ld_pos ^ (key & 15)) * 8, dst + i * 1024);
            }
        }
    };
    auto issue_v = [&](int tile) {
        const uint32_t dst = lds0 + 2 * KBYTES + (tile & 1) * VBYTES + wave_s * 4096;
        if (tile * BC + BC <= Sk) {
            const unsigned char* src = (const unsigned char*)V + (long long)(tile * BC + 16 * wave_s) * v_row_bytes;
#pragma unroll
            for (int i = 0; i < 4; i++) attn_dma16_base(src + 4 * i * v_row_bytes, v_lane_off[i & 1], dst + i * 1024);
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int key = 4 * (wave * 4 + i) + ld_key;
                const int gkey = min(tile * BC + key, Sk - 1);
                attn_dma16(V + (long long)gkey * a.vs[2] + (ld_pos ^ (((key & 3) << 2) ^ (((key >> 2) & 1) << 1))) * 8, dst + i * 1024);
            }
        }
    };

    // Q fragments (B operand of S^T = K Q^T): lane (l16, g) holds row 16 qb + l16, elements 32 ks + 8 g .. + 7, scaled
    const int qrow0 = q0 + wave * 32 + l16;
    u32x4 qf[2][4];
#pragma unroll
    for (int qb = 0; qb < 2; qb++)
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
            const int row = qrow0 + 16 * qb;
            u32x4 z = {0u, 0u, 0u, 0u};
            qf[qb][ks] = row < a.Sq ? scale_frag<T>(*(const u32x4*)(Q + (long long)row * a.qs[2] + 32 * ks + 8 * g), sl2) : z;
        }

    // tiles of the workgroup, units (32 keys) of this wave
    int ntiles = (Sk + BC - 1) / BC;
    if (a.causal) {
        long long lastkey = (long long)q0 + BR - 1 + qoff;
        if (lastkey < 0) ntiles = 0;
        else { long long nt = lastkey / BC + 1; if (nt < ntiles) ntiles = (int)nt; }
    }
    const int wq_min = q0 + wave_s * 32, wq_max = wq_min + 31;
    auto key_limit = [&](int q) -> int {        // last key query q may see (sequence end and causal diagonal in one bound)
        long long lim = Sk - 1;
        if (a.causal) { long long c = (long long)q + qoff; if (c < lim) lim = c; }
        return (int)(lim < -1 ? -1 : lim);
    };
    int nu = 0;
    if (wq_min < a.Sq) nu = (key_limit(wq_max) + 1 + 31) / 32;
    if (nu > 2 * ntiles) nu = 2 * ntiles;
    nu = __builtin_amdgcn_readfirstlane(nu);
    // a unit all of whose keys every row of the wave sees needs no mask: units 0 .. ufull
    const int ufull = __builtin_amdgcn_readfirstlane((key_limit(wq_min) + 1) / 32 - 1);
    const int usteady = min(nu - 2, ufull);          // units 1 .. usteady take the interleaved block
    int klim[2];                                      // element (kb, r) of unit u is masked when 32 u + 16 kb + r > klim
#pragma unroll
    for (int qb = 0; qb < 2; qb++) klim[qb] = key_limit(qrow0 + 16 * qb) - 4 * g;

    // LDS read addresses (per lane, stage 0; the stage bit 14 is toggled at every tile barrier)
    //   K fragment (block kb of the unit, k-step ks): key 16 kb + l16, chunk 4 ks + g  ->  base ^ (ks << 6), + kb * 4096
    //   V^T fragment (block db): two transposing reads, lane addresses key 16 q + 4 g + l16 / 4, the 8 bytes at head-dim
    //   16 db + 4 (l16 % 4)  ->  base ^ (db << 5), + q * 4096; it receives keys 16 q + 4 g .. + 3 of head-dim 16 db + l16
    uint32_t k_ad[4], v_ad[8];
    {
        const uint32_t k_lane = l16 * 256 + ((g ^ l16) << 4);
        const int vr = 4 * g + (l16 >> 2);
        const uint32_t v_swz = (((vr & 3) << 2) ^ (((vr >> 2) & 1) << 1)) | ((l16 >> 1) & 1);
        const uint32_t v_lane = vr * 256 + (v_swz << 4) + (l16 & 1) * 8;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) k_ad[ks] = (lds0 + k_lane) ^ (uint32_t)(ks << 6);
        // V addresses start at stage 1: the first barrier moves them to stage 0, where tile 0 lands
#pragma unroll
        for (int db = 0; db < 8; db++) v_ad[db] = ((lds0 + 2 * KBYTES + v_lane) ^ (uint32_t)(db << 5)) ^ (uint32_t)VBYTES;
    }
    auto k_frag = [&](int ub, int kb, int ks) -> u32x4 {
        return *(const __attribute__((address_space(3))) u32x4*)(k_ad[ks] + (2 * ub + kb) * 4096);
    };
    auto v_frag = [&](int ub, int db) -> u32x4 {
        const uint32_t ad = v_ad[db] + ub * 8192;
        u32x2 w0 = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4a*)ad));
        u32x2 w1 = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4a*)(ad + 4096)));
        return u32x4{w0[0], w0[1], w1[0], w1[1]};
    };

    f32x4a oacc[8][2];
#pragma unroll
    for (int db = 0; db < 8; db++)
#pragma unroll
        for (int qb = 0; qb < 2; qb++) oacc[db][qb] = f32x4a{0.0f, 0.0f, 0.0f, 0.0f};
    f32x4a sacc[2][2][2];          // [unit parity][kb][qb]: exp2 arguments (scaled logit minus the row's reference)
    u32x4 pf[2][2];                // [unit parity][qb]: packed probabilities, the B operand of the P V step
#pragma unroll
    for (int p = 0; p < 2; p++)
#pragma unroll
        for (int x = 0; x < 2; x++) {
            pf[p][x] = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
            for (int y = 0; y < 2; y++) sacc[p][x][y] = f32x4a{0.0f, 0.0f, 0.0f, 0.0f};
        }
    f32x4a minit[2] = {f32x4a{0.0f, 0.0f, 0.0f, 0.0f}, f32x4a{0.0f, 0.0f, 0.0f, 0.0f}};      // -m_ref, the start value of an S block
    float m_ref[2] = {0.0f, 0.0f}, l_run[2] = {0.0f, 0.0f};
    bool first = true;
    u32x4 kfr[4], vfr[4];          // fragment rings of the interleaved block (carried from a B block into the next A block)
#pragma unroll
    for (int i = 0; i < 4; i++) { kfr[i] = u32x4{0u, 0u, 0u, 0u}; vfr[i] = u32x4{0u, 0u, 0u, 0u}; }

    // ---- plain (not interleaved) forms of the three steps of a unit
    auto qk_plain = [&](auto par_c, int ub) {                  // S(parity) of the unit at half ub of the tile k_ad points to
        constexpr int par = decltype(par_c)::value;
#pragma unroll
        for (int ks = 0; ks < 4; ks++)
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
                const u32x4 kf = k_frag(ub, kb, ks);
#pragma unroll
                for (int qb = 0; qb < 2; qb++)
                    sacc[par][kb][qb] = MmaX16<T>::run(kf, qf[qb][ks], ks == 0 ? minit[qb] : sacc[par][kb][qb]);
            }
    };
    auto pv_plain = [&](auto par_c, int ub) {                  // O += V^T P(parity)^T, unit at half ub of the tile v_ad points to
        constexpr int par = decltype(par_c)::value;
#pragma unroll
        for (int db = 0; db < 8; db++) {
            const u32x4 vf = v_frag(ub, db);
#pragma unroll
            for (int qb = 0; qb < 2; qb++) oacc[db][qb] = MmaX16<T>::run(vf, pf[par][qb], oacc[db][qb]);
        }
    };
    // probabilities of unit u (parity par) with the row maxima formed first: the reference of a row moves when this is the
    // wave's first unit or the row's maximum lies more than 8 above it; O, l, this unit's (and, when next_valid, the next
    // unit's) exponents move with it.  Adds the unit's row sums to l.
    auto softmax_exact = [&](auto par_c, int u, bool apply_mask, bool next_valid) {
        constexpr int par = decltype(par_c)::value;
        if (apply_mask) {
#pragma unroll
            for (int qb = 0; qb < 2; qb++) {
                const int rel = klim[qb] - 32 * u;
#pragma unroll
                for (int kb = 0; kb < 2; kb++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (16 * kb + r > rel) sacc[par][kb][qb][r] = -INFINITY;
            }
        }
        float mx[2];
        bool need[2];
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
            float m = fmaxf(fmaxf(sacc[par][0][qb][0], sacc[par][0][qb][1]), fmaxf(sacc[par][0][qb][2], sacc[par][0][qb][3]));
            m = fmaxf(m, fmaxf(fmaxf(sacc[par][1][qb][0], sacc[par][1][qb][1]), fmaxf(sacc[par][1][qb][2], sacc[par][1][qb][3])));
            m = fmaxf(m, shfl_xor_f(m, 16));
            m = fmaxf(m, shfl_xor_f(m, 32));
            mx[qb] = m;
            need[qb] = (first || m > 8.0f) && m > -INFINITY && m < INFINITY;
        }
        if (__builtin_amdgcn_ballot_w64(need[0] || need[1]) != 0ull) {
#pragma unroll
            for (int qb = 0; qb < 2; qb++) {
                const float delta = need[qb] ? mx[qb] : 0.0f;
                const float alpha = __builtin_amdgcn_exp2f(-delta);
                m_ref[qb] += delta;
                l_run[qb] *= alpha;
                const float nm = -m_ref[qb];
                minit[qb] = f32x4a{nm, nm, nm, nm};
#pragma unroll
                for (int db = 0; db < 8; db++)
#pragma unroll
                    for (int r = 0; r < 4; r++) oacc[db][qb][r] *= alpha;
#pragma unroll
                for (int kb = 0; kb < 2; kb++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        sacc[par][kb][qb][r] -= delta;
                        if (next_valid) sacc[par ^ 1][kb][qb][r] -= delta;
                    }
            }
        }
        first = false;
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
            float ps = 0.0f;
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int rp = 0; rp < 2; rp++) {
                    const uint32_t pk = pack2_p<T>(__builtin_amdgcn_exp2f(sacc[par][kb][qb][2 * rp]),
                                                   __builtin_amdgcn_exp2f(sacc[par][kb][qb][2 * rp + 1]));
                    ps = add_pair<T>(pk, ps);
                    pf[par][qb][2 * kb + rp] = pk;
                }
            l_run[qb] += ps;
        }
    };

    // ---- the interleaved block of unit u (1 <= u <= usteady): P(u-1) V and S(u+1) on the matrix pipe, exp2 / convert / row
    // sum of unit u beside them.  ISB: second half of a tile (after the barrier): issues the tile loads, starts with cold
    // fragment rings and leaves them filled for the block that follows; the first-half form finds them filled.
    auto steady = [&](auto par_c, auto isb_c, int u, int tile_k, int tile_v) {
        constexpr int par = decltype(par_c)::value;
        constexpr bool ISB = decltype(isb_c)::value;
        // this block's units inside their tiles: P V reads half (u - 1) & 1, S reads half (u + 1) & 1
        constexpr int ub_v = ISB ? 0 : 1, ub_k = ISB ? 0 : 1;
        if (ISB) {
#pragma unroll
            for (int i = 0; i < 3; i++) { vfr[i] = v_frag(ub_v, i); kfr[i] = k_frag(ub_k, i & 1, i >> 1); }
        }
        const unsigned char* ksrc = nullptr; const unsigned char* vsrc = nullptr;
        uint32_t kdst = 0, vdst = 0;
        bool dma_k = false, dma_v = false;
        if (ISB) {
            dma_k = tile_k >= 0 && tile_k * BC + BC <= Sk;
            dma_v = tile_v >= 0 && tile_v * BC + BC <= Sk;
            if (tile_k >= 0 && !dma_k) issue_k(tile_k);
            if (tile_v >= 0 && !dma_v) issue_v(tile_v);
            ksrc = (const unsigned char*)K + (long long)(tile_k * BC + 16 * wave_s) * k_row_bytes;
            vsrc = (const unsigned char*)V + (long long)(tile_v * BC + 16 * wave_s) * v_row_bytes;
            kdst = lds0 + (tile_k & 1) * KBYTES + wave_s * 4096;
            vdst = lds0 + 2 * KBYTES + (tile_v & 1) * VBYTES + wave_s * 4096;
        }
        float ps[2] = {0.0f, 0.0f};
        float e0 = 0.0f, e1 = 0.0f;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < 16; s++) {
            const int db = s >> 1, qb = s & 1;
            const int f = s >> 1, ks = f >> 1, kb = f & 1;
            // fragment reads three ahead; past the end of this block (ISB only) they are the first ones of the next block
            if (qb == 0) {
                if (db + 3 < 8) vfr[(db + 3) & 3] = v_frag(ub_v, db + 3);
                else if (ISB) vfr[(db + 3) & 3] = v_frag(1, db + 3 - 8);
                if (f + 3 < 8) kfr[(f + 3) & 3] = k_frag(ub_k, (f + 3) & 1, (f + 3) >> 1);
                else if (ISB) kfr[(f + 3) & 3] = k_frag(1, (f + 3 - 8) & 1, (f + 3 - 8) >> 1);
            }
            oacc[db][qb] = MmaX16<T>::run(vfr[db & 3], pf[par ^ 1][qb], oacc[db][qb]);
            sacc[par ^ 1][kb][qb] = MmaX16<T>::run(kfr[f & 3], qf[qb][ks], ks == 0 ? minit[qb] : sacc[par ^ 1][kb][qb]);
            if (ISB && s < 8) {
                if (s < 4) { if (dma_k) attn_dma16_base(ksrc + 4 * s * k_row_bytes, k_lane_off[s], kdst + s * 1024); }
                else { if (dma_v) attn_dma16_base(vsrc + 4 * (s - 4) * v_row_bytes, v_lane_off[s & 1], vdst + (s - 4) * 1024); }
            }
            // logit pair pi of unit u: even slots the two exponentials, odd slots convert + row sum
            const int pi = s >> 1, pq = pi >> 2, pkb = (pi >> 1) & 1, prp = pi & 1;
            if ((s & 1) == 0) {
                e0 = __builtin_amdgcn_exp2f(sacc[par][pkb][pq][2 * prp]);
                e1 = __builtin_amdgcn_exp2f(sacc[par][pkb][pq][2 * prp + 1]);
                asm volatile("" : "+v"(e0), "+v"(e1));
            } else {
                uint32_t pk = pack2_p<T>(e0, e1);
                ps[pq] = add_pair<T>(pk, ps[pq]);
                asm volatile("" : "+v"(pk), "+v"(ps[pq]));
                pf[par][pq][2 * pkb + prp] = pk;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if (__builtin_amdgcn_ballot_w64(!(ps[0] < BIG) || !(ps[1] < BIG)) != 0ull) {
            // a probability left the range of exp2 against the standing reference: form this unit again with its row maxima
            softmax_exact(par_c, u, false, true);
        } else {
            l_run[0] += ps[0];
            l_run[1] += ps[1];
        }
    };

    // one unit iteration: P(u-1) V, softmax of unit u, S(u+1); tile_k / tile_v: tiles whose loads a second-half iteration issues
    auto iteration = [&](auto par_c, auto isb_c, int u, int tile_k, int tile_v) {
        constexpr int par = decltype(par_c)::value;
        constexpr bool ISB = decltype(isb_c)::value;
        if (u >= 1 && u <= usteady) { steady(par_c, isb_c, u, tile_k, tile_v); return; }
        if (ISB) {
            if (tile_k >= 0) issue_k(tile_k);
            if (tile_v >= 0) issue_v(tile_v);
        }
        if (u >= 1 && u - 1 < nu) pv_plain(std::integral_constant<int, par ^ 1>{}, ISB ? 0 : 1);
        if (u < nu) softmax_exact(par_c, u, u > ufull, false);
        if (u + 1 < nu) qk_plain(std::integral_constant<int, par ^ 1>{}, ISB ? 0 : 1);
    };

    // ---- pipeline: loads of K(0), V(0), K(1); S(0); then per tile  A(t) | barrier, loads of K(t+2) and V(t+1) | B(t)
    if (ntiles > 0) { issue_k(0); issue_v(0); }
    if (ntiles > 1) issue_k(1);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (nu > 0) qk_plain(std::integral_constant<int, 0>{}, 0);
    for (int tl = 0; tl < ntiles; tl++) {
        iteration(std::integral_constant<int, 0>{}, std::false_type{}, 2 * tl, -1, -1);
        __builtin_amdgcn_s_waitcnt(0);      // this wave's loads of K(t+1) and V(t) have landed ...
        __syncthreads();                    // ... everyone's have, and everyone is done with K(t) and V(t-1)
#pragma unroll
        for (int ks = 0; ks < 4; ks++) k_ad[ks] ^= (uint32_t)KBYTES;
#pragma unroll
        for (int db = 0; db < 8; db++) v_ad[db] ^= (uint32_t)VBYTES;
        iteration(std::integral_constant<int, 1>{}, std::true_type{}, 2 * tl + 1, tl + 2 < ntiles ? tl + 2 : -1, tl + 1 < ntiles ? tl + 1 : -1);
    }
    if (2 * ntiles - 1 < nu && ntiles > 0) pv_plain(std::integral_constant<int, 1>{}, 1);      // P V of the last unit

    // ---- epilogue: row sums over the four lanes of a query, normalise, store
    float inv[2], l_tot[2];
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
        float l = l_run[qb];
        l += shfl_xor_f(l, 16);
        l += shfl_xor_f(l, 32);
        l_tot[qb] = l;
        inv[qb] = l > 0.0f ? 1.0f / l : 0.0f;
    }
    if (a.lse && g == 0) {
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
            const int qi = qrow0 + 16 * qb;
            if (qi < a.Sq) a.lse[(long long)bh * a.Sq + qi] = l_tot[qb] > 0.0f ? (m_ref[qb] + __builtin_amdgcn_logf(l_tot[qb])) * LN2 : -INFINITY;
        }
    }
    if (Elem<OutT>::BYTES == 4 && a.vec_out) {
        // fp32 O through LDS: a lane holds 16-byte pieces of its rows; staged per wave as [32 rows][512 B] (chunk c of row r at
        // position c ^ r) and written back as whole 512-byte rows with non-temporal stores (O is written once and would
        // otherwise displace K and V tiles that other workgroups re-read).  Every wave is past its last LDS read of the
        // tiles only after a barrier.
        __syncthreads();
        unsigned char* stg = smem + wave * 16384;
#pragma unroll
        for (int qb = 0; qb < 2; qb++)
#pragma unroll
            for (int db = 0; db < 8; db++) {
                const int r = 16 * qb + l16, c = 4 * db + g;
                *(f32x4*)(stg + r * 512 + ((c ^ r) << 4)) =
                    f32x4{oacc[db][qb][0] * inv[qb], oacc[db][qb][1] * inv[qb], oacc[db][qb][2] * inv[qb], oacc[db][qb][3] * inv[qb]};
            }
        const int c = lane & 31;
#pragma unroll
        for (int q = 0; q < 16; q++) {
            const int r = 2 * q + (lane >> 5);
            const int row = q0 + wave * 32 + r;
            const f32x4 v = *(const f32x4*)(stg + r * 512 + ((c ^ r) << 4));
            f32x4* dst = (f32x4*)((float*)a.o + b * a.os[0] + hd * a.os[1] + (long long)row * a.os[2] + c * 4);
            if (row < a.Sq) __builtin_nontemporal_store(v, dst);
        }
    } else {
        typedef typename Raw2<OutT>::type out_t;
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
            const int qi = qrow0 + 16 * qb;
            if (qi < a.Sq) {
                out_t* __restrict__ O = (out_t*)a.o + b * a.os[0] + hd * a.os[1] + (long long)qi * a.os[2];
#pragma unroll
                for (int db = 0; db < 8; db++) {
                    const int d0 = 16 * db + 4 * g;
                    const float v0 = oacc[db][qb][0] * inv[qb], v1 = oacc[db][qb][1] * inv[qb];
                    const float v2 = oacc[db][qb][2] * inv[qb], v3 = oacc[db][qb][3] * inv[qb];
                    if constexpr (Elem<OutT>::BYTES == 4) {
                        O[d0] = as_u32(v0); O[d0 + 1] = as_u32(v1); O[d0 + 2] = as_u32(v2); O[d0 + 3] = as_u32(v3);
                    } else {
                        const uint32_t w0 = Elem<OutT>::narrow(v0) | (Elem<OutT>::narrow(v1) << 16);
                        const uint32_t w1 = Elem<OutT>::narrow(v2) | (Elem<OutT>::narrow(v3) << 16);
                        if (a.vec_out) *(u32x2*)(O + d0) = u32x2{w0, w1};
                        else { O[d0] = (out_t)(w0 & 0xFFFFu); O[d0 + 1] = (out_t)(w0 >> 16); O[d0 + 2] = (out_t)(w1 & 0xFFFFu); O[d0 + 3] = (out_t)(w1 >> 16); }
                    }
                }
            }
        }
    }
    if (npass > 1) __syncthreads();      // the next pass's loads must not overtake this pass's last LDS reads
    }   // pass
}

template <typename T, typename OutT>
static hipError_t launch_x16(AttnArgs a, hipStream_t stream)
{
    auto kern = attn_fwd_x16_kernel<T, OutT>;
    constexpr int smem = 2 * (64 * 256 + 64 * 256);
    static unsigned long long attr_done = 0;
    if (hipError_t e = ensure_dynamic_smem((const void*)kern, smem, &attr_done)) return e;
    a.qtiles = (a.Sq + 127) / 128;
    // causal self-attention with an even number of query tiles: tile i and tile qtiles-1-i in one workgroup (equal work everywhere)
    a.paired = (a.causal && a.qoff == 0 && a.Sq == a.Sk && a.qtiles >= 2 && a.qtiles % 2 == 0) ? 1 : 0;
    const long long nblk = (long long)(a.paired ? a.qtiles / 2 : a.qtiles) * a.B * a.H;
    if (nblk > 0x7FFFFFFFLL || nblk <= 0) return hipErrorInvalidValue;
    hipLaunchKernelGGL(kern, dim3((unsigned)nblk), dim3(256), smem, stream, a);
    return hipGetLastError();
}

hipError_t launch_attn_x16(int kind, int out16, AttnArgs a, hipStream_t stream)
{
    if (a.D != 128 || a.nsplit > 1 || a.part || a.stream || a.bt || !(a.scale > 0.0f)) return hipErrorInvalidValue;
    if (kind == 1) return out16 ? launch_x16<f16_t, f16_t>(a, stream) : launch_x16<f16_t, float>(a, stream);
    if (kind == 2) return out16 ? launch_x16<bf16_t, bf16_t>(a, stream) : launch_x16<bf16_t, float>(a, stream);
    return hipErrorInvalidValue;
}

}  // namespace aidn
