// Fused attention forward for the 16-bit types at head dimension 128 (plain or causal, aligned contiguous K/V), software-pipelined:
// the prefill form of FlashAttentionV2 / ScaledDotProductAttention behind the reference's backend slot
// (src/AiDotNet.Tensors/Engines/DirectGpu/HIP/HipBackend.cs:6118-6302; value semantics
// src/AiDotNet.Tensors/Engines/CpuEngine.cs:29146-29288, update order Engines/Simd/FusedAttention.cs:159-286).
//
// Workgroup: 128 query rows of one (batch, head), four waves of 32 rows; K and V stream through LDS as 64-key tiles (direct
// global -> LDS loads, two stages each, one barrier per tile) and are consumed in units of 32 keys.  Formulation and LDS layouts
// are those of attn_fwd_dl_kernel (attention.hip): S^T = K Q^T and O^T += V^T P^T on v_mfma_f32_32x32x16, lane (l32, h) holds
// query l32 and keys 8 (r / 4) + 4 h + r % 4 of a unit, P^T in accumulator order is the B operand of the P V step.
//
// What differs is the order of the work.
//   * Unit u's exponentials run beside the matrix work of its neighbours: one iteration issues P(u-1) V and S(u+1) = K(u+1) Q^T
//     as one stream of 16 MFMAs (alternating, so the dependent S chain is spaced) with exp2 / convert / row sum of unit u spread
//     one logit pair per two MFMAs.  Matrix and vector instructions of an iteration are independent of each other.  (With this
//     instruction shape a vector instruction issued behind an MFMA costs the matrix pipe nothing up to about three per MFMA;
//     measured on the part: 16.8 cycles per 16 cycles of matrix work with one exp2, one plain vector instruction and one 16-byte
//     LDS read per MFMA, against 22 with v_mfma_f32_16x16x32, whose issue leaves no such room.)
//   * No running-maximum pass: the reference m of a row only has to keep exp2 in range, it need not be the maximum
//     (LSE = m + log2(l) holds for any m; O = acc / l does not depend on it).  It is set from the row maximum of the wave's first
//     unit and then stands; a unit's probabilities are formed against it at once and the unit's sum tells whether one of them
//     left the range.  Only then, and in the units at the two ends of a wave's key range (first unit, masked units), the row
//     maxima are formed and O, l and m moved.  Per logit that leaves one FMA, one v_exp_f32, half a packed convert, half a v_dot2.
//   * LDS fragment reads run RING - 1 MFMAs ahead of their use through a register ring that is carried from the second half of
//     a tile into the first half of the next.
#include "attention_common.hpp"
#ifdef PREFILL_LOOP_FILE
#include PREFILL_LOOP_FILE
#else
#include "attention_prefill_loop.inc"
#endif

namespace aidn {

#define PREFILL_HEAD_GROUP 4
#ifndef PREFILL_RING
#define PREFILL_RING 4
#endif

template <typename T, typename OutT>
__global__ __launch_bounds__(256, 2) void attn_prefill_kernel(const AttnArgs a)
{
    typedef uint16_t raw_t;
    constexpr int BC = 64, BR = 128, R = PREFILL_RING;
    constexpr int KBYTES = BC * 256, VBYTES = BC * 256;
    constexpr float BIG = 1.152921504606847e18f;       // 2^60: a unit's probability sum beyond it means exp2 left the range
    static_assert(16 % R == 0 && R >= 2, "the fragment ring is indexed i % R over the 16 MFMAs of an iteration");

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int l32 = lane & 31, h = lane >> 5;
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
            // heads in groups of PREFILL_HEAD_GROUP (their K and V are what an XCD's L2 holds); a group's query tiles heaviest first
            const bool whole = rem == 0 && per % a.qtiles == 0;
            const int heads = whole ? per / a.qtiles : nblk / a.qtiles;
            const int at = whole ? idx : logical;
            const int gsz = heads < PREFILL_HEAD_GROUP ? heads : PREFILL_HEAD_GROUP;
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

    // Direct-to-LDS loads.  This wave's share of a tile: K wave-loads 4 w .. 4 w + 3 and the same of V, each 4 keys x 256 B; lane ->
    // (key = 4 * load + lane / 16, chunk position lane % 16).  LDS layout [key][256 B]: 16-byte chunk c of key k sits at position
    // c ^ (k & 15) in a K tile (b128 fragment reads) and at c ^ ((k & 3) << 2) in a V tile (transposing reads).
    const int ld_key = lane >> 4, ld_pos = lane & 15;
    const long long k_row_bytes = a.ks[2] * 2, v_row_bytes = a.vs[2] * 2;
    // (wave-load i of K differs from load 0 by the swizzle bits 4 i of the chunk position: an XOR with i << 6 when the row pitch
    // is a multiple of 256 bytes, which the launcher checks)
    const uint32_t k_lane_off = (uint32_t)(ld_key * k_row_bytes) + ((ld_pos ^ ld_key) << 4);
    const uint32_t v_lane_off = (uint32_t)(ld_key * v_row_bytes) + ((ld_pos ^ (ld_key << 2)) << 4);

    const int npass = a.paired ? 2 : 1;
    for (int pass = 0; pass < npass; pass++) {
#ifdef PREFILL_DBG
    unsigned long long stamp[8];
#define STAMP(i) stamp[i] = __builtin_amdgcn_s_memtime()
    STAMP(0);
#else
#define STAMP(i)
#endif
    if (pass == 1) qt = a.qtiles - 1 - qt;
    const int b = bh / a.H, hd = bh - b * a.H;
    const int kvh = hd / (a.H / a.Hkv);
    const int q0 = qt * BR;
    const int qi = q0 + wave * 32 + l32;
    const raw_t* __restrict__ Q = (const raw_t*)a.q + b * a.qs[0] + hd * a.qs[1];
    const raw_t* __restrict__ K = (const raw_t*)a.k + b * a.ks[0] + kvh * a.ks[1];
    const raw_t* __restrict__ V = (const raw_t*)a.v + b * a.vs[0] + kvh * a.vs[1];

    auto issue_k = [&](int tile) {
        const uint32_t dst = lds0 + (tile & 1) * KBYTES + wave_s * 4096;
        if (tile * BC + BC <= Sk) {
            const unsigned char* src = (const unsigned char*)K + (long long)(tile * BC + 16 * wave_s) * k_row_bytes;
#pragma unroll
            for (int i = 0; i < 4; i++) attn_dma16_base(src + 4 * i * k_row_bytes, k_lane_off ^ (uint32_t)(i << 6), dst + i * 1024);
        } else {
            // (the lane index is taken through an opaque copy: nothing of this rare path is then computed ahead of the loops)
            int ln = lane;
            asm volatile("" : "+v"(ln));
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int key = 4 * (wave_s * 4 + i) + (ln >> 4);       // key inside the tile
                const int gkey = min(tile * BC + key, Sk - 1);          // rows past the end are clamped loads, masked later
                attn_dma16(K + (long long)gkey * a.ks[2] + ((ln & 15) ^ (key & 15)) * 8, dst + i * 1024);
            }
        }
    };
    auto issue_v = [&](int tile) {
        const uint32_t dst = lds0 + 2 * KBYTES + (tile & 1) * VBYTES + wave_s * 4096;
        if (tile * BC + BC <= Sk) {
            const unsigned char* src = (const unsigned char*)V + (long long)(tile * BC + 16 * wave_s) * v_row_bytes;
#pragma unroll
            for (int i = 0; i < 4; i++) attn_dma16_base(src + 4 * i * v_row_bytes, v_lane_off, dst + i * 1024);
        } else {
            int ln = lane;
            asm volatile("" : "+v"(ln));
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int key = 4 * (wave_s * 4 + i) + (ln >> 4);
                const int gkey = min(tile * BC + key, Sk - 1);
                attn_dma16(V + (long long)gkey * a.vs[2] + ((ln & 15) ^ ((key & 3) << 2)) * 8, dst + i * 1024);
            }
        }
    };

    // Q fragments (B operand of S^T = K Q^T): lane (l32, h) holds row l32, elements 16 s + 8 h .. + 7
    u32x4 qf[8];
#pragma unroll
    for (int s = 0; s < 8; s++) {
        u32x4 z = {0u, 0u, 0u, 0u};
        qf[s] = (qi < a.Sq) ? *(const u32x4*)(Q + (long long)qi * a.qs[2] + (2 * s + h) * 8) : z;
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
    const int klim = key_limit(qi) - 4 * h;          // element r of unit u is masked when 32 u + 8 (r / 4) + r % 4 > klim

    // LDS read addresses (per lane).  The two stages of the K tiles are 32 KB of four 32-key units, unit index j at offset
    // (j % 4) * 8 KB, and so are the V tiles: the K and the V addresses each point at one unit and move to the next one by an
    // XOR (8 KB when leaving an even unit, 24 KB when leaving an odd one).
    //   K fragment (k-step s of the unit): key l32, chunk (2 s + h) ^ (key & 15); the upper four k-steps by an XOR of bit 7
    //   V^T fragment (s = 4 * (16-key half) + head-dim block): two transposing reads 8 keys apart; in a 16-lane group lane j
    //   addresses key 4 h + j / 4 and the 8 bytes at head-dim 4 (j % 4) of its 16-wide block
    uint32_t k_ad[4], v_ad[4];
    int k_unit = 0, v_unit = 0;
    {
        // (from an opaque copy of the lane index, so that these are formed here, per pass, rather than kept across the passes)
        int ln = lane;
        asm volatile("" : "+v"(ln));
        const int jl = ln & 15, l32p = ln & 31, hp = ln >> 5;
        const uint32_t k_lane = l32p * 256 + ((hp ^ (l32p & 15)) << 4);
        const uint32_t v_lane = (4 * hp + (jl >> 2)) * 256 + ((16 * ((ln >> 4) & 1) + 4 * (jl & 3)) >> 3) * 16 + (jl & 1) * 8 + ((jl >> 2) << 6);
#pragma unroll
        for (int s = 0; s < 4; s++) k_ad[s] = (lds0 + k_lane) ^ (uint32_t)(s << 5);
#pragma unroll
        for (int i = 0; i < 4; i++) v_ad[i] = (lds0 + 2 * KBYTES + v_lane) ^ (uint32_t)(i << 6);
    }
    auto next_k_unit = [&]() {
        const uint32_t x = (k_unit & 1) ? 24576u : 8192u;
#pragma unroll
        for (int s = 0; s < 4; s++) k_ad[s] ^= x;
        k_unit++;
    };
    auto next_v_unit = [&]() {
        const uint32_t x = (v_unit & 1) ? 24576u : 8192u;
#pragma unroll
        for (int i = 0; i < 4; i++) v_ad[i] ^= x;
        v_unit++;
    };
    auto k_frag = [&](int s) -> u32x4 {
        return *(const __attribute__((address_space(3))) u32x4*)(s < 4 ? k_ad[s] : (k_ad[s - 4] ^ 128u));
    };
    auto v_frag = [&](int s) -> u32x4 {
        const uint32_t ad = v_ad[s & 3] + 16 * (s >> 2) * 256;
        u32x2 w0 = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4a*)ad));
        u32x2 w1 = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4a*)(ad + 8 * 256)));
        return u32x4{w0[0], w0[1], w1[0], w1[1]};
    };

    f32x16 oacc[4];
    f32x16 sacc;                   // logits of one unit (S^T accumulator layout), then its exponentials in place
    u32x4 pf[2];                   // [16-key half]: packed probabilities of one unit, the B operand of the P V step
    float m_ref = -INFINITY;       // reference point of the exponent (log2 domain); the same in lanes l and l ^ 32
    float l_run = 0.0f;
    u32x4 fr[R];                   // fragment ring of the interleaved block, carried from block to block

    // ---- plain (not interleaved) forms of the three steps of a unit
    auto qk_plain = [&]() {                                    // S of the unit the K addresses point to
#pragma unroll
        for (int r = 0; r < 16; r++) sacc[r] = 0.0f;
#pragma unroll
        for (int s = 0; s < 8; s++) {
            Mma32<T>::run(sacc, k_frag(s), qf[s]);
            if (s & 1) __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto pv_plain = [&]() {                                    // O += V^T P^T, unit the V addresses point to
#pragma unroll
        for (int s = 0; s < 8; s++) {
            Mma32<T>::run(oacc[s & 3], v_frag(s), pf[s >> 2]);
            if (s & 1) __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto mask_unit = [&](int u) {
        const int rel = klim - 32 * u;
#pragma unroll
        for (int r = 0; r < 16; r++)
            if (8 * (r >> 2) + (r & 3) > rel) sacc[r] = -INFINITY;
    };
    // Probabilities of unit u with the row maxima formed first (the safe form, also the wave's first unit in the fast form): the
    // reference of a row is raised when the row's maximum lies more than 8 above it (always on first use).  Adds the row sums to l.
    auto softmax_exact = [&](int u, bool apply_mask) {
        if (apply_mask) mask_unit(u);
        float m = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; r++) m = fmaxf(m, sacc[r]);
        const float mloc = max_with_partner32(m) * sl2;            // scale > 0: max commutes with the scaling
        if (__builtin_amdgcn_ballot_w64(mloc > m_ref + 8.0f) != 0ull) {
            const float m_new = (mloc > m_ref + 8.0f && mloc < INFINITY) ? mloc : m_ref;
            const float alpha = (m_new == -INFINITY) ? 1.0f : __builtin_amdgcn_exp2f(m_ref - m_new);
            m_ref = m_new;
            l_run *= alpha;
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int r = 0; r < 16; r++) oacc[i][r] *= alpha;
        }
        const float m_use = (m_ref == -INFINITY) ? 0.0f : m_ref;
        float ps = 0.0f;
#pragma unroll
        for (int pi = 0; pi < 8; pi++) {
            const float p0 = __builtin_amdgcn_exp2f(fmaf(sacc[2 * pi], sl2, -m_use));
            const float p1 = __builtin_amdgcn_exp2f(fmaf(sacc[2 * pi + 1], sl2, -m_use));
            const uint32_t pk = pack2_p<T>(p0, p1);
            ps = add_pair<T>(pk, ps);
            pf[pi >> 2][pi & 3] = pk;
        }
        l_run += ps;
    };
    // what every wave does once per unit whether it computes or not: before an odd unit the loads of K(t+2) and V(t+1) (t = u / 2:
    // the tiles they replace went out of use at the barrier just passed), after an even unit the barrier that publishes K(t+1), V(t)
    auto unit_loads = [&](int u) {
        const int tl = u >> 1;
        if (tl + 2 < ntiles) issue_k(tl + 2);
        if (tl + 1 < ntiles) issue_v(tl + 1);
    };
    auto tile_barrier = [&]() {
        __builtin_amdgcn_s_waitcnt(0);      // this wave's loads have landed, its fragment reads are in registers ...
        __syncthreads();                    // ... everyone's
    };

    // ---- the interleaved block of unit u (sacc holds S(u), pf holds P(u-1), the V addresses point at unit u-1, the K addresses at
    // unit u+1, the ring holds the first R-1 fragments): the matrix pipe runs P(u-1) V, then S(u+1); beside the first the vector
    // pipe turns the logits of unit u into exponentials in place (FMA + exp2 against the standing reference, two logits per MFMA);
    // between the two it packs them into the P buffer, which the P V step has finished reading, and sums them; S(u+1) then lands
    // in the registers the logits have left.  Once the block's last fragment read is issued the addresses move on, an even unit
    // passes the tile barrier, and the reads that follow fetch the first fragments of the next block.  An odd unit issues the tile
    // loads (dma) one per MFMA.  Returns the unit's row sums.
    auto full_block = [&](int u, bool dma) -> float {
        // fragment stream of the block: V^T fragments 0 .. 7, then K fragments 0 .. 7
        auto frag = [&](int j) -> u32x4 { return j < 8 ? v_frag(j) : k_frag(j - 8); };
        const int tile_k = (u >> 1) + 2, tile_v = (u >> 1) + 1;
        const unsigned char* ksrc = (const unsigned char*)K + (long long)(tile_k * BC + 16 * wave_s) * k_row_bytes;
        const unsigned char* vsrc = (const unsigned char*)V + (long long)(tile_v * BC + 16 * wave_s) * v_row_bytes;
        const uint32_t kdst = lds0 + (tile_k & 1) * KBYTES + wave_s * 4096;
        const uint32_t vdst = lds0 + 2 * KBYTES + (tile_v & 1) * VBYTES + wave_s * 4096;
        const float m_use = (m_ref == -INFINITY) ? 0.0f : m_ref;
        float ps = 0.0f;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            if (i == 16 - (R - 1)) {
                // every fragment of this block is requested: on to the next units
                next_k_unit();
                next_v_unit();
                if (!(u & 1)) tile_barrier();
                __builtin_amdgcn_sched_barrier(0);
            }
            // the fragment R - 1 MFMAs ahead; past the end of this block it is one of the first of the next block
            fr[(i + R - 1) % R] = frag((i + R - 1) % 16);
            if (i < 8) {
                Mma32<T>::run(oacc[i & 3], fr[i % R], pf[i >> 2]);
                float e0 = __builtin_amdgcn_exp2f(fmaf(sacc[2 * i], sl2, -m_use));
                float e1 = __builtin_amdgcn_exp2f(fmaf(sacc[2 * i + 1], sl2, -m_use));
                asm volatile("" : "+v"(e0), "+v"(e1));
                sacc[2 * i] = e0;
                sacc[2 * i + 1] = e1;
                if (dma) {
                    if (i < 4) attn_dma16_base(ksrc + 4 * i * k_row_bytes, k_lane_off ^ (uint32_t)(i << 6), kdst + i * 1024);
                    else attn_dma16_base(vsrc + 4 * (i - 4) * v_row_bytes, v_lane_off, vdst + (i - 4) * 1024);
                }
            } else {
                const int s = i - 8;
                if (s == 0) {
                    // every P V MFMA has been issued: P(u) takes the buffer, then S(u+1) the registers of the exponentials
#pragma unroll
                    for (int pi = 0; pi < 8; pi++) {
                        uint32_t pk = pack2_p<T>(sacc[2 * pi], sacc[2 * pi + 1]);
                        ps = add_pair<T>(pk, ps);
                        pf[pi >> 2][pi & 3] = pk;
                    }
                    asm volatile("" : "+v"(ps));
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int r = 0; r < 16; r++) sacc[r] = 0.0f;
                }
                Mma32<T>::run(sacc, fr[i % R], qf[s]);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        return ps;
    };

    // The workgroup's loads: K(0), V(0), K(1) up front; before every odd unit K(t+2) and V(t+1), after every even unit the tile
    // barrier.  Fast form: unit 0 is done in plain steps (its row maxima set the reference of every row), units 1 .. take the
    // interleaved block, which forms the probabilities against that standing reference.  Should a probability leave the range of
    // exp2 (seen in the row sums at the end), the pass is run again in the safe form, which forms the row maxima of every unit.
    uint32_t* const redo_flag = (uint32_t*)smem;       // one word per wave, in the tile memory once the tiles are done with
    const int nunits = 2 * ntiles;
    for (int attempt = 0; attempt < 2; attempt++) {
    const bool safe = attempt == 1;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[i][r] = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; r++) sacc[r] = 0.0f;
    pf[0] = u32x4{0u, 0u, 0u, 0u}; pf[1] = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int i = 0; i < R; i++) fr[i] = u32x4{0u, 0u, 0u, 0u};
    m_ref = -INFINITY; l_run = 0.0f;
    while (k_unit & 3) next_k_unit();           // (a second attempt starts from unit 0 again)
    while (v_unit & 3) next_v_unit();
    k_unit = 0; v_unit = 0;
    if (ntiles > 0) { issue_k(0); issue_v(0); }
    if (ntiles > 1) issue_k(1);
    tile_barrier();
    STAMP(1);
    if (nu > 0) qk_plain();                     // S(0)
    next_k_unit();
    if (!safe) {
        if (nu > 0) softmax_exact(0, 0 > ufull);                // P(0); sets the reference of every row
        if (nu > 1) qk_plain();                                 // S(1)
        next_k_unit();                                          // K addresses at unit 2, V addresses at unit 0: block 1 may start
        if (nunits > 1) {
            __syncthreads();                                    // everyone is done with the first half of K(0), which K(2) replaces
            if (1 < nu) {
#pragma unroll
                for (int j = 0; j < R - 1; j++) fr[j] = v_frag(j);
            }
        }
        // Runs of whole unmasked units go through the assembly form of the block (attention_prefill_loop.inc: the same steps, every
        // LDS offset an immediate, no instruction that is not needed).  run_units(u, n, loads): units u .. u + n - 1 with sacc, pf,
        // the addresses and l as the C++ block would find and leave them; the first k_loads / v_loads odd units of the run issue the
        // loads of K(t+2) / V(t+1), which have to be whole tiles.
        auto run_units = [&](int u, int n, int k_loads, int v_loads) {
            typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));
            typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
            u32x16 qlo, qhi;
#pragma unroll
            for (int s4 = 0; s4 < 4; s4++)
#pragma unroll
                for (int e = 0; e < 4; e++) { qlo[4 * s4 + e] = qf[s4][e]; qhi[4 * s4 + e] = qf[4 + s4][e]; }
            // read addresses of unit 0 (the K addresses stand at unit u + 1, the V addresses at unit u - 1)
            const uint32_t koff = (uint32_t)((u + 1) & 3) << 13, voff = (uint32_t)((u - 1) & 3) << 13;
            const u32x4 kad0 = {k_ad[0] ^ koff, k_ad[1] ^ koff, k_ad[2] ^ koff, k_ad[3] ^ koff};
            const u32x4 kad1 = {kad0[0] ^ 128u, kad0[1] ^ 128u, kad0[2] ^ 128u, kad0[3] ^ 128u};
            const u32x4 vad = {v_ad[0] ^ voff, v_ad[1] ^ voff, v_ad[2] ^ voff, v_ad[3] ^ voff};
            const u32x4 klo = {k_lane_off, k_lane_off ^ 64u, k_lane_off ^ 128u, k_lane_off ^ 192u};
            const uint32_t vlo = v_lane_off;
            const float negm = (m_ref == -INFINITY) ? -0.0f : -m_ref;
            float ps = 0.0f;
            const int tl = u >> 1;
            unsigned long long kptr = (unsigned long long)(uintptr_t)((const unsigned char*)K + (long long)((tl + 2) * BC + 16 * wave_s) * k_row_bytes);
            unsigned long long vptr = (unsigned long long)(uintptr_t)((const unsigned char*)V + (long long)((tl + 1) * BC + 16 * wave_s) * v_row_bytes);
            const unsigned long long ktile = (unsigned long long)(BC * k_row_bytes), vtile = (unsigned long long)(BC * v_row_bytes);
            const u32x8 sc = {(uint32_t)(4 * k_row_bytes), (uint32_t)(4 * v_row_bytes), (uint32_t)ktile, (uint32_t)(ktile >> 32),
                              (uint32_t)vtile, (uint32_t)(vtile >> 32), lds0 + wave_s * 4096u, lds0 + 2 * KBYTES + wave_s * 4096u};
            const float sl2s = sl2;
            int count = __builtin_amdgcn_readfirstlane(n);
            int kleft = __builtin_amdgcn_readfirstlane(k_loads), vleft = __builtin_amdgcn_readfirstlane(v_loads);
            const int phase = __builtin_amdgcn_readfirstlane((u - 1) & 3);
            u32x4 p0 = pf[0], p1 = pf[1];
#define PREFILL_LOOP_OPERANDS \
                : "+{v[0:15]}"(oacc[0]), "+{v[16:31]}"(oacc[1]), "+{v[32:47]}"(oacc[2]), "+{v[48:63]}"(oacc[3]), "+{v[64:79]}"(sacc), \
                  "+{v[80:83]}"(p0), "+{v[84:87]}"(p1), "+{v170}"(ps), "+{s[40:41]}"(kptr), "+{s[42:43]}"(vptr), "+{s53}"(count), "+{s57}"(kleft), "+{s58}"(vleft) \
                : "{v[88:103]}"(qlo), "{v[104:119]}"(qhi), "{v[152:155]}"(kad0), "{v[156:159]}"(kad1), "{v[160:163]}"(vad), \
                  "{v[164:167]}"(klo), "{v168}"(vlo), "{v169}"(negm), "{s[44:51]}"(sc), "{s52}"(sl2s), "{s56}"(phase) \
                : "v120", "v121", "v122", "v123", "v124", "v125", "v126", "v127", "v128", "v129", "v130", "v131", "v132", "v133", "v134", \
                  "v135", "v136", "v137", "v138", "v139", "v140", "v141", "v142", "v143", "v144", "v145", "v146", "v147", "v148", "v149", \
                  "v150", "v151", "v172", "v173", "v176", "v177", "v178", "v179", "v180", "v181", "v182", "v183", "v184", "v185", "v186", \
                  "v187", "v188", "v189", "v190", "v191", "s54", "s55", "scc", "vcc", "memory"
            if constexpr (std::is_same<T, f16_t>::value) asm volatile(PREFILL_LOOP_F16 PREFILL_LOOP_OPERANDS);
            else asm volatile(PREFILL_LOOP_BF16 PREFILL_LOOP_OPERANDS);
#undef PREFILL_LOOP_OPERANDS
            pf[0] = p0; pf[1] = p1;
            l_run += ps;
            for (int i = 0; i < (n & 3); i++) { next_k_unit(); next_v_unit(); }
            k_unit += n & ~3; v_unit += n & ~3;
        };
        int u_first = 1;
        STAMP(2);
        {
            // one run: units 1 .. u_last, whole, unmasked, with a successor; it ends ahead of the odd unit that would have to load a
            // partial tile (the last tile of a sequence that is not a multiple of 64 keys long)
            const int whole = min(ntiles, Sk / BC);                 // the workgroup's tiles 0 .. whole - 1 are whole tiles
            int u_last = min(ufull, nu - 1);
            if (whole < ntiles) u_last = min(u_last, 2 * (whole - 2));      // unit 2 (whole - 2) + 1 loads tile `whole` as its K tile
            if (u_last >= 1) {
                // odd unit 2 t + 1 loads K(t + 2) for t <= whole - 3 and V(t + 1) for t <= whole - 2
                run_units(1, u_last, max(0, whole - 2), max(0, whole - 1));
                u_first = u_last + 1;
                if (u_first < nu) {
#pragma unroll
                    for (int j = 0; j < R - 1; j++) fr[j] = v_frag(j);
                }
            }
        }
        STAMP(3);
        for (int u = u_first; u < nunits; u++) {
            const int tl = u >> 1;
            const bool fast_loads = (u & 1) && tl + 2 < ntiles && (tl + 2) * BC + BC <= Sk && (tl + 1) * BC + BC <= Sk;
            if ((u & 1) && !fast_loads) unit_loads(u);
            if (u < nu) {
                if (u > ufull) mask_unit(u);
                l_run += full_block(u, fast_loads);
            } else {
                if (u == nu) pv_plain();
                next_k_unit();
                next_v_unit();
                if ((u & 1) && fast_loads) unit_loads(u);
                if (!(u & 1)) tile_barrier();
            }
        }
        if (nunits == nu && nunits > 0) pv_plain();             // P V of the workgroup's last unit
        STAMP(4);
        const bool left_range = __builtin_amdgcn_ballot_w64(!(l_run < 1.2676506e30f)) != 0ull;
        __syncthreads();                        // every wave is past its last fragment read
        if (lane == 0) redo_flag[wave] = left_range ? 1u : 0u;
        __syncthreads();
        const bool redo = (redo_flag[0] | redo_flag[1] | redo_flag[2] | redo_flag[3]) != 0u;
#ifdef PREFILL_NO_REDO
        break;
#endif
        if (!redo) break;
        __syncthreads();                        // everyone has read the flags before the next attempt's loads land on them
    } else {
        // K addresses at unit 1, V addresses at unit 0
        for (int u = 0; u < nunits; u++) {
            if (u & 1) unit_loads(u);
            if (u >= 1) {
                if (u - 1 < nu) pv_plain();
                next_v_unit();
            }
            if (u < nu) softmax_exact(u, u > ufull);
            if (u + 1 < nu) qk_plain();
            next_k_unit();
            if (!(u & 1)) tile_barrier();
        }
        if (nunits - 1 < nu && nunits > 0) pv_plain();
    }
    }   // attempt

    // ---- epilogue: normalise, store
    STAMP(5);
    const float l_tot = sum_with_partner32(l_run);
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    if (Elem<OutT>::BYTES == 4 && a.vec_out) {
        // fp32 O through LDS: the lane holds 16-byte pieces of ONE row (64 rows per store instruction, each a partial line); staged
        // per wave as [32 rows][512 B] (chunk c of row r at position c ^ r, conflict-free both ways) and written back as whole
        // 512-byte rows with non-temporal stores (O is written once and would otherwise displace K and V tiles that other
        // workgroups re-read).  The tile memory is free only when every wave is past its last fragment read: barrier first.
        __syncthreads();
        unsigned char* stg = smem + wave_s * 16384;
        int lnw = lane;
        asm volatile("" : "+v"(lnw));
        const int l32w = lnw & 31, hw = lnw >> 5;
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int c = 8 * i + 2 * g + hw;
                *(f32x4*)(stg + l32w * 512 + ((c ^ l32w) << 4)) =
                    f32x4{oacc[i][4 * g + 0] * inv, oacc[i][4 * g + 1] * inv, oacc[i][4 * g + 2] * inv, oacc[i][4 * g + 3] * inv};
            }
        if (a.lse && h == 0 && qi < a.Sq)
            a.lse[(long long)bh * a.Sq + qi] = l_tot > 0.0f ? (m_ref + __builtin_amdgcn_logf(l_tot)) * LN2 : -INFINITY;
        // (row and chunk from an opaque copy of the lane index: the store addresses are then formed here, not ahead of the loops)
        int lne = lane;
        asm volatile("" : "+v"(lne));
        const int c = lne & 31;
#pragma unroll
        for (int q = 0; q < 16; q++) {
            const int r = 2 * q + (lne >> 5);
            const int row = q0 + wave_s * 32 + r;
            const f32x4 v = *(const f32x4*)(stg + r * 512 + ((c ^ r) << 4));
            f32x4* dst = (f32x4*)((float*)a.o + b * a.os[0] + hd * a.os[1] + (long long)row * a.os[2] + c * 4);
            if (row < a.Sq) __builtin_nontemporal_store(v, dst);
        }
    } else if (qi < a.Sq) {
        typedef typename Raw2<OutT>::type out_t;
        out_t* __restrict__ O = (out_t*)a.o + b * a.os[0] + hd * a.os[1] + (long long)qi * a.os[2];
#pragma unroll
        for (int i = 0; i < 4; i++) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int d0 = i * 32 + 8 * g + 4 * h;
                const float v0 = oacc[i][4 * g + 0] * inv, v1 = oacc[i][4 * g + 1] * inv;
                const float v2 = oacc[i][4 * g + 2] * inv, v3 = oacc[i][4 * g + 3] * inv;
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
        if (a.lse && h == 0)
            a.lse[(long long)bh * a.Sq + qi] = l_tot > 0.0f ? (m_ref + __builtin_amdgcn_logf(l_tot)) * LN2 : -INFINITY;
    }
    STAMP(6);
#ifdef PREFILL_DBG
    __builtin_amdgcn_s_waitcnt(0);
    STAMP(7);
    {
        float dv = (float)(stamp[0] & 0xFFFFFFull);
#pragma unroll
        for (int i = 1; i < 8; i++) if (lane == i) dv = (float)(long long)(stamp[i] - stamp[i - 1]);
        if (a.lse && lane < 8) a.lse[(long long)bh * a.Sq + q0 + wave_s * 32 + lane] = dv;
    }
#endif
    if (npass > 1) __syncthreads();      // the next pass's loads must not overtake this pass's last LDS reads
    }   // pass
}

template <typename T, typename OutT>
static hipError_t launch_prefill(AttnArgs a, hipStream_t stream)
{
    auto kern = attn_prefill_kernel<T, OutT>;
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

hipError_t launch_attn_prefill(int kind, int out16, AttnArgs a, hipStream_t stream)
{
    if (a.D != 128 || a.nsplit > 1 || a.part || a.stream || a.bt || !(a.scale > 0.0f)) return hipErrorInvalidValue;
    if ((a.ks[2] * 2) % 256 != 0) return hipErrorInvalidValue;      // the lane offsets of the K wave-loads are formed by XOR
    if (kind == 1) return out16 ? launch_prefill<f16_t, f16_t>(a, stream) : launch_prefill<f16_t, float>(a, stream);
    if (kind == 2) return out16 ? launch_prefill<bf16_t, bf16_t>(a, stream) : launch_prefill<bf16_t, float>(a, stream);
    return hipErrorInvalidValue;
}

}  // namespace aidn
