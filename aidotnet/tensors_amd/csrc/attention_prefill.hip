// The software-pipelined prefill kernel of attention_prefill.hip on v_mfma_f32_16x16x32 (same workgroup, tile loads, LDS layouts,
// standing exponent reference with a safe second form, resident workgroups that take their passes in turn): fused attention forward
// for the 16-bit types at head dimension 128 on dense arrays, behind the reference's FlashAttentionV2 / ScaledDotProductAttention
// slot (src/AiDotNet.Tensors/Engines/DirectGpu/HIP/HipBackend.cs:6118-6302; value semantics
// src/AiDotNet.Tensors/Engines/CpuEngine.cs:29146-29288, update order Engines/Simd/FusedAttention.cs:159-286).
//
// Why a second instruction shape: the kernel runs at the board's power limit (1.33-1.37 kW of 1.4 kW at 1.76-1.83 GHz), where what
// counts is the energy a flop takes, and the 16 x 16 x 32 shape moves half the accumulator registers per flop of the 32 x 32 x 16
// one (the same loop with every MFMA replaced by two of this shape on the same operand registers ran 6-7 % faster).
//
// A wave's 32 queries are two blocks of 16 (qb), a unit's 32 keys two blocks of 16 (kb), the head dimension eight blocks of 16
// (db).  Lane (c, g) = (lane % 16, lane / 16):
//   S^T block (kb, qb) = K_kb Q_qb^T: the lane holds query c of the block and keys 4 g + r, r = 0..3 (accumulator layout);
//   P^T of a query block as the B operand of P V: the lane's k-positions 8 g + e, e = 4 kb + r, ARE its eight probabilities
//     in accumulator order (key 16 kb + 4 g + r), so P goes from the exponentials to the operand by packed converts alone,
//     and the V^T fragment presents the keys in that order (two transposing reads: keys 4 g .. + 3 and 16 + 4 g .. + 3);
//   O^T block (db, qb) += V^T_db P^T_qb: the lane holds query c and head-dim 16 db + 4 g + r.
// Every fragment read from LDS (a K block of one 32-wide k-step, a V^T d-block) feeds two MFMAs, one per query block.
#include "attention_common.hpp"
#ifdef PREFILL_LOOP_FILE
#include PREFILL_LOOP_FILE
#else
#ifndef PREFILL_LOOP_INC
#define PREFILL_LOOP_INC "attention_prefill_loop.inc"
#endif
#include PREFILL_LOOP_INC
#endif

namespace aidn {

#define PREFILL_HEAD_GROUP 4
#ifndef PREFILL_EXTRA_LDS
#define PREFILL_EXTRA_LDS 0      // (timing experiments: more than 12 KB extra leaves one workgroup per CU)
#endif

template <typename T, typename OutT>
__global__ __launch_bounds__(256, 2) void attn_prefill_kernel(const AttnArgs a)
{
    typedef uint16_t raw_t;
    constexpr int BC = 64, BR = 128;
    constexpr int KBYTES = BC * 256, VBYTES = BC * 256;
    constexpr float BIG = 1.152921504606847e18f;       // 2^60: a unit's probability sum beyond it means exp2 left the range

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int c16 = lane & 15, g4 = lane >> 4;
    // The grid is at most two workgroups per CU; a workgroup takes the virtual blocks blockIdx.x, blockIdx.x + gridDim.x, ... one
    // after the other (so that the loads that open a pass can be issued while the pass before it is still storing), and, with
    // paired causal query tiles, two passes per virtual block.  Item k of this workgroup -> (batch * head, query tile):
    const int npass = a.paired ? 2 : 1;
    auto decode = [&](int k, int& bh, int& qt) {
        int nblk = a.nvb, pid = blockIdx.x + (k >> (npass - 1)) * gridDim.x;
        int per = nblk >> 3, rem = nblk & 7;
        int xcd = pid & 7, idx = pid >> 3;
        int logical = (xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per) + idx;
        bh = (int)fastdiv((uint32_t)logical, a.dqtiles);
        qt = a.qtiles - 1 - (logical - bh * a.qtiles);
        if (a.paired) {
            // XCD-contiguous heads, qtiles / 2 workgroups per head: first the late (heavy) tile of the pair, then the early one
            const int units = a.qtiles >> 1;
            bh = (int)fastdiv((uint32_t)logical, a.dunits);
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
        if (npass == 2 && (k & 1)) qt = a.qtiles - 1 - qt;
    };
    const bool alt_flavour = (int)blockIdx.x >= a.alt_from;
    const int nitems = (int)blockIdx.x < a.nvb ? ((a.nvb - 1 - (int)blockIdx.x) / (int)gridDim.x + 1) * npass : 0;

    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)smem);
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    const float sl2 = a.scale * LOG2E;
    const int Sk = a.Sk;
    const int qoff = a.qoff;                    // (the launcher keeps |qoff|, Sq and Sk below 2^30: row and key sums stay 32-bit)

    // Direct-to-LDS loads.  This wave's share of a tile: K wave-loads 4 w .. 4 w + 3 and the same of V, each 4 keys x 256 B; lane ->
    // (key = 4 * load + lane / 16, chunk position lane % 16).  LDS layout [key][256 B]: 16-byte chunk c of key k sits at position
    // c ^ (k & 15) in a K tile (b128 fragment reads) and at c ^ ((k & 3) << 2) ^ ((k >> 2 & 1) << 1) in a V tile (transposing reads:
    // a half-wave reads eight keys, 4 g .. 4 g + 7, 32 bytes each, and the position spreads them over all 64 banks).
    const int ld_key = lane >> 4, ld_pos = lane & 15;
    // Q, K, V and O are dense [batch, head, row, 128] arrays (the launcher checks): row r of (batch, head) pair j is row
    // j * rows + r of the array, 256 bytes a row in the 16-bit types.
    constexpr int k_row_bytes = 256, v_row_bytes = 256;
    // (wave-load i of K differs from load 0 by the swizzle bits 4 i of the chunk position: an XOR with i << 6)
    const uint32_t k_lane_off = (uint32_t)(ld_key * k_row_bytes) + ((ld_pos ^ ld_key) << 4);
    const uint32_t v_lane_off = (uint32_t)(ld_key * v_row_bytes) + ((ld_pos ^ (ld_key << 2)) << 4);

    // tiles of the workgroup whose first query row is q0
    auto tiles_of = [&](int q0) -> int {
        int nt = (Sk + BC - 1) / BC;
        if (a.causal) {
            const int lastkey = q0 + BR - 1 + qoff;
            if (lastkey < 0) nt = 0;
            else { const int c = lastkey / BC + 1; if (c < nt) nt = c; }
        }
        return nt;
    };
    auto issue_k = [&](const uint16_t* K, int tile) {
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
                attn_dma16(K + (long long)gkey * 128 + ((ln & 15) ^ (key & 15)) * 8, dst + i * 1024);
            }
        }
    };
    auto issue_v = [&](const uint16_t* V, int tile) {
        const uint32_t dst = lds0 + 2 * KBYTES + (tile & 1) * VBYTES + wave_s * 4096;
        if (tile * BC + BC <= Sk) {
            const unsigned char* src = (const unsigned char*)V + (long long)(tile * BC + 16 * wave_s) * v_row_bytes;
#pragma unroll
            for (int i = 0; i < 4; i++) attn_dma16_base(src + 4 * i * v_row_bytes, v_lane_off ^ (uint32_t)((i & 1) << 5), dst + i * 1024);
        } else {
            int ln = lane;
            asm volatile("" : "+v"(ln));
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int key = 4 * (wave_s * 4 + i) + (ln >> 4);
                const int gkey = min(tile * BC + key, Sk - 1);
                attn_dma16(V + (long long)gkey * 128 + ((ln & 15) ^ ((key & 3) << 2) ^ (((key >> 2) & 1) << 1)) * 8, dst + i * 1024);
            }
        }
    };
    // What opens a pass and can be asked for while the pass before it is still storing: the Q fragments (B operand of
    // S^T = K Q^T) and the K tiles 0 and 1, which land in the K half of the
    // tile memory (the stores stage through the V half).
    typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));
    u32x16 qlo, qhi;                        // query block 0 and 1, four k-steps each (held the way the assembly loop takes them)
    auto qfrag = [&](int qb, int ks) -> u32x4 {
        return qb == 0 ? u32x4{qlo[4 * ks], qlo[4 * ks + 1], qlo[4 * ks + 2], qlo[4 * ks + 3]}
                       : u32x4{qhi[4 * ks], qhi[4 * ks + 1], qhi[4 * ks + 2], qhi[4 * ks + 3]};
    };
    // (B operand of S^T = K Q^T: lane (c, g) holds query c of the block, elements 32 ks + 8 g .. + 7)
    auto open_pass = [&](int bh, int qt) {
        int ln = lane;
        asm volatile("" : "+v"(ln));
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
            // (a lane whose row lies past the end of the sequence takes the last row: what it computes is never stored)
            const int qrow = min(qt * BR + wave_s * 32 + 16 * qb + (ln & 15), a.Sq - 1);
            const uint16_t* Q = (const uint16_t*)a.q + ((long long)(bh * a.Sq) << 7) + qrow * 128 + (ln >> 4) * 8;
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                const u32x4 x = *(const u32x4*)(Q + 32 * ks);
#pragma unroll
                for (int e = 0; e < 4; e++) { if (qb == 0) qlo[4 * ks + e] = x[e]; else qhi[4 * ks + e] = x[e]; }
            }
        }
        // (H = Hkv * group: K/V head b Hkv + head / group is (b H + head) / group)
        const uint16_t* K = (const uint16_t*)a.k + ((long long)((int)fastdiv((uint32_t)bh, a.dgroup) * Sk) << 7);
        const int nt = tiles_of(qt * BR);
        if (nt > 0) issue_k(K, 0);
        if (nt > 1) issue_k(K, 1);
    };

    int bh = 0, qt = 0;
    if (nitems > 0) { decode(0, bh, qt); open_pass(bh, qt); }
    for (int item = 0; item < nitems; item++) {
    const int pass = item & 1;
#ifdef PREFILL_DBG
    unsigned long long stamp[12];
#define STAMP(i) stamp[i] = __builtin_amdgcn_s_memtime()
    STAMP(0);
#else
#define STAMP(i)
#endif
    const int q0 = qt * BR;
    const int qi[2] = {q0 + wave * 32 + c16, q0 + wave * 32 + 16 + c16};
    const long long kv_first = (long long)((int)fastdiv((uint32_t)bh, a.dgroup) * Sk) << 7;      // first element of the head's K and V
    const raw_t* __restrict__ K = (const raw_t*)a.k + kv_first;
    const raw_t* __restrict__ V = (const raw_t*)a.v + kv_first;

    // tiles of the workgroup, units (32 keys) of this wave
    const int ntiles = tiles_of(q0);
    const int wq_min = q0 + wave_s * 32, wq_max = wq_min + 31;
    auto key_limit = [&](int q) -> int {        // last key query q may see (sequence end and causal diagonal in one bound)
        int lim = Sk - 1;
        if (a.causal) { const int c = q + qoff; if (c < lim) lim = c; }
        return lim < -1 ? -1 : lim;
    };
    int nu = 0;
    if (wq_min < a.Sq) nu = (key_limit(wq_max) + 1 + 31) / 32;
    if (nu > 2 * ntiles) nu = 2 * ntiles;
    nu = __builtin_amdgcn_readfirstlane(nu);
    // a unit all of whose keys every row of the wave sees needs no mask: units 0 .. ufull
    const int ufull = __builtin_amdgcn_readfirstlane((key_limit(wq_min) + 1) / 32 - 1);
    // element r of S^T block (kb, qb) in unit u is masked when 32 u + 16 kb + r > klim[qb]
    const int klim[2] = {key_limit(qi[0]) - 4 * g4, key_limit(qi[1]) - 4 * g4};

    // LDS read addresses (per lane).  The two stages of the K tiles are 32 KB of four 32-key units, unit index j at offset
    // (j % 4) * 8 KB, and so are the V tiles: the K and the V addresses each point at one unit and move to the next one by an
    // XOR (8 KB when leaving an even unit, 24 KB when leaving an odd one).
    //   K fragment (block kb, k-step ks): key 16 kb + c, chunk (4 ks + g) ^ c; the k-steps differ by an XOR of bits 6-7, kb by 4 KB
    //   V^T fragment of d-block db: two transposing reads 16 keys apart; in the 16-lane group g lane c addresses key 4 g + c / 4 and
    //   the 8 bytes at head-dim 4 (c % 4) of the block; the d-blocks differ by an XOR of bits 5-7
    uint32_t k_ad[4], v_ad[8];
    int k_unit = 0, v_unit = 0;
    {
        // (from an opaque copy of the lane index, so that these are formed here, per pass, rather than kept across the passes)
        int ln = lane;
        asm volatile("" : "+v"(ln));
        const int cp = ln & 15, gp = ln >> 4;
        const uint32_t k_lane = cp * 256 + ((gp ^ cp) << 4);
        const uint32_t v_lane = (4 * gp + (cp >> 2)) * 256 + ((((cp & 3) >> 1) ^ (((cp >> 2) & 3) << 2) ^ ((gp & 1) << 1)) << 4) + (cp & 1) * 8;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) k_ad[ks] = (lds0 + k_lane) ^ (uint32_t)(ks << 6);
#pragma unroll
        for (int j = 0; j < 8; j++) v_ad[j] = (lds0 + 2 * KBYTES + v_lane) ^ (uint32_t)(j << 5);
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
        for (int i = 0; i < 8; i++) v_ad[i] ^= x;
        v_unit++;
    };
    auto k_frag = [&](int kb, int ks) -> u32x4 {
        return *(const __attribute__((address_space(3))) u32x4*)(k_ad[ks] + kb * 4096);
    };
    auto v_frag = [&](int db) -> u32x4 {
        const uint32_t ad = v_ad[db];
        u32x2 w0 = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4a*)ad));
        u32x2 w1 = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4a*)(ad + 16 * 256)));
        return u32x4{w0[0], w0[1], w1[0], w1[1]};
    };
    auto mma16 = [&](f32x4 acc, const u32x4& x, const u32x4& y) -> f32x4 {
        if constexpr (std::is_same<T, f16_t>::value)
            return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, x), __builtin_bit_cast(f16x8, y), acc, 0, 0, 0);
        else
            return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, x), __builtin_bit_cast(bf16x8, y), acc, 0, 0, 0);
    };

    // (sixteen-register groups, the way the assembly loop takes them: O block (db, qb) is elements 4 ((2 db + qb) % 4) .. + 3 of
    // oacc[db / 2], logit block (kb, qb) elements 4 (2 kb + qb) .. + 3 of sacc)
    f32x16 oacc[4];
    f32x16 sacc;                   // logits of one unit, then its exponentials in place
    u32x4 pf[2];                   // [query block]: packed probabilities of one unit, the B operand of the P V step
    float m_ref[2] = {-INFINITY, -INFINITY};   // per query block: reference point of the exponent (log2 domain); the same in the four lanes of a query
    float l_run[2] = {0.0f, 0.0f};
    auto get4 = [&](const f32x16& v, int at) -> f32x4 { return f32x4{v[4 * at], v[4 * at + 1], v[4 * at + 2], v[4 * at + 3]}; };
    auto put4 = [&](f32x16& v, int at, const f32x4& x) { v[4 * at] = x[0]; v[4 * at + 1] = x[1]; v[4 * at + 2] = x[2]; v[4 * at + 3] = x[3]; };
    // a value of the four lanes (g = 0..3) that share a query: maximum / sum over them
    // (two lane-swap instructions of the vector pipe each, no trip through the LDS crossbar)
    auto max_over_g = [&](float v) -> float { return max_with_partner32(max_with_partner16(v)); };
    auto sum_over_g = [&](float v) -> float { return sum_with_partner32(sum_with_partner16(v)); };

    // ---- plain (not interleaved) forms of the three steps of a unit
    auto qk_plain = [&]() {                                    // S of the unit the K addresses point to
#pragma unroll
        for (int r = 0; r < 16; r++) sacc[r] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
#pragma unroll
            for (int kb = 0; kb < 2; kb++) {
                const u32x4 kf = k_frag(kb, ks);
#pragma unroll
                for (int qb = 0; qb < 2; qb++) put4(sacc, 2 * kb + qb, mma16(get4(sacc, 2 * kb + qb), kf, qfrag(qb, ks)));
            }
            if (ks == 1) __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto pv_plain = [&]() {                                    // O += V^T P^T, unit the V addresses point to
#pragma unroll
        for (int db = 0; db < 8; db++) {
            const u32x4 vf = v_frag(db);
#pragma unroll
            for (int qb = 0; qb < 2; qb++) put4(oacc[db >> 1], (2 * db + qb) & 3, mma16(get4(oacc[db >> 1], (2 * db + qb) & 3), vf, pf[qb]));
            if (db == 3) __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto mask_unit = [&](int u) {
#pragma unroll
        for (int t = 0; t < 16; t++) {
            const int kb = t >> 3, qb = (t >> 2) & 1, r = t & 3;
            if (16 * kb + r > klim[qb] - 32 * u) sacc[t] = -INFINITY;
        }
    };
    // Probabilities of unit u with the row maxima formed first (the safe form, also the wave's first unit in the fast form): the
    // reference of a row is raised when the row's maximum lies more than 8 above it (always on first use).  Adds the row sums to l.
    auto softmax_exact = [&](int u, bool apply_mask, const bool first) {
        if (apply_mask) mask_unit(u);
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
            float m = -INFINITY;
#pragma unroll
            for (int kb = 0; kb < 2; kb++)
#pragma unroll
                for (int r = 0; r < 4; r++) m = fmaxf(m, sacc[8 * kb + 4 * qb + r]);
            const float mloc = max_over_g(m) * sl2;                    // scale > 0: max commutes with the scaling
            if (first) {
                m_ref[qb] = mloc < INFINITY ? mloc : -INFINITY;        // nothing accumulated yet: no O or l to move
            } else {
                // (the accumulators are scaled whether a reference moves or not, by 1 if not: a branch around the scaling costs
                // more, in copies of all of them, than the scaling)
                const float m_new = (mloc > m_ref[qb] + 8.0f && mloc < INFINITY) ? mloc : m_ref[qb];
                const float alpha = (m_new == -INFINITY) ? 1.0f : __builtin_amdgcn_exp2f(m_ref[qb] - m_new);
                m_ref[qb] = m_new;
                l_run[qb] *= alpha;
#pragma unroll
                for (int db = 0; db < 8; db++)
#pragma unroll
                    for (int r = 0; r < 4; r++) oacc[db >> 1][4 * ((2 * db + qb) & 3) + r] *= alpha;
            }
            const float m_use = (m_ref[qb] == -INFINITY) ? 0.0f : m_ref[qb];
            float ps = 0.0f;
#pragma unroll
            for (int e2 = 0; e2 < 4; e2++) {
                const int t0 = 8 * (e2 >> 1) + 4 * qb + 2 * (e2 & 1);
                const float p0 = __builtin_amdgcn_exp2f(fmaf(sacc[t0], sl2, -m_use));
                const float p1 = __builtin_amdgcn_exp2f(fmaf(sacc[t0 + 1], sl2, -m_use));
                const uint32_t pk = pack2_p<T>(p0, p1);
                ps = add_pair<T>(pk, ps);
                pf[qb][e2] = pk;
            }
            l_run[qb] += ps;
        }
    };
    // what every wave does once per unit whether it computes or not: before an odd unit the loads of K(t+2) and V(t+1) (t = u / 2:
    // the tiles they replace went out of use at the barrier just passed), after an even unit the barrier that publishes K(t+1), V(t)
    auto unit_loads = [&](int u) {
        const int tl = u >> 1;
        if (tl + 2 < ntiles) issue_k(K, tl + 2);
        if (tl + 1 < ntiles) issue_v(V, tl + 1);
    };
    auto tile_barrier = [&]() {
        __builtin_amdgcn_s_waitcnt(0);      // this wave's loads have landed, its fragment reads are in registers ...
        __syncthreads();                    // ... everyone's
    };

    // The workgroup's loads: K(0), V(0), K(1) up front; before every odd unit K(t+2) and V(t+1), after every even unit the tile
    // barrier.  Fast form: unit 0 is done in plain steps (its row maxima set the reference of every row), units 1 .. take the
    // interleaved block, which forms the probabilities against that standing reference.  Should a probability leave the range of
    // exp2 (seen in the row sums at the end), the pass is run again in the safe form, which forms the row maxima of every unit.
    // Runs of whole unmasked units go through the assembly form of the block (attention_prefill_loop.inc: the same steps, every
    // LDS offset an immediate, no instruction that is not needed).  run_units(u, n, loads): units u .. u + n - 1 with sacc, pf,
    // the addresses and l as the C++ block would find and leave them; the first k_loads / v_loads odd units of the run issue the
    // loads of K(t+2) / V(t+1), which have to be whole tiles.
    auto run_units = [&](int u, int n, int k_loads, int v_loads, bool masked_last) {
        typedef uint32_t u32x8 __attribute__((ext_vector_type(8)));
        // read addresses of unit 0 (the K addresses stand at unit u + 1, the V addresses at unit u - 1)
        const uint32_t koff = (uint32_t)((u + 1) & 3) << 13, voff = (uint32_t)((u - 1) & 3) << 13;
        const u32x4 kad = {k_ad[0] ^ koff, k_ad[1] ^ koff, k_ad[2] ^ koff, k_ad[3] ^ koff};
        const u32x4 vad0 = {v_ad[0] ^ voff, v_ad[1] ^ voff, v_ad[2] ^ voff, v_ad[3] ^ voff};
        const u32x4 vad1 = {v_ad[4] ^ voff, v_ad[5] ^ voff, v_ad[6] ^ voff, v_ad[7] ^ voff};
        const u32x4 klo = {k_lane_off, k_lane_off ^ 64u, k_lane_off ^ 128u, k_lane_off ^ 192u};
        const uint32_t vlo = v_lane_off, vlo_odd = v_lane_off ^ 32u;
        const float negm0 = (m_ref[0] == -INFINITY) ? -0.0f : -m_ref[0], negm1 = (m_ref[1] == -INFINITY) ? -0.0f : -m_ref[1];
        float ps0 = 0.0f, ps1 = 0.0f;
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
        // (with masked_last the run is n whole units and then unit u + n, masked first; n >= 1)
        int mask_follows = __builtin_amdgcn_readfirstlane(masked_last ? 1 : 0);
        const int mask_rel0 = klim[0] - 32 * (u + n), mask_rel1 = klim[1] - 32 * (u + n);
        const float ninf = -INFINITY;
        // (the routine has two flavours that differ in the wave priority of every other unit: the workgroups of the second half of a
        // resident grid share their CUs with those of the first half and take the other flavour, so the two take turns in leading)
        const int flavour = __builtin_amdgcn_readfirstlane(alt_flavour ? 1 : 0);
        if (masked_last) n++;
        u32x4 p0 = pf[0], p1 = pf[1];
#define PREFILL_LOOP_OPERANDS \
            : "+{v[0:15]}"(oacc[0]), "+{v[16:31]}"(oacc[1]), "+{v[32:47]}"(oacc[2]), "+{v[48:63]}"(oacc[3]), "+{v[64:79]}"(sacc), \
              "+{v[80:83]}"(p0), "+{v[84:87]}"(p1), "+{v167}"(ps0), "+{v168}"(ps1), "+{s[40:41]}"(kptr), "+{s[42:43]}"(vptr), "+{s53}"(count), "+{s57}"(kleft), "+{s58}"(vleft), "+{s59}"(mask_follows) \
            : "{v[88:103]}"(qlo), "{v[104:119]}"(qhi), "{v[152:155]}"(kad), "{v[192:195]}"(vad0), "{v[196:199]}"(vad1), \
              "{v[160:163]}"(klo), "{v164}"(vlo), "{v174}"(vlo_odd), "{v165}"(negm0), "{v166}"(negm1), "{s[44:51]}"(sc), "{s52}"(sl2s), "{s56}"(phase), "{s60}"(flavour), \
              "{v171}"(mask_rel0), "{v172}"(mask_rel1), "{v173}"(ninf) \
            : "v120", "v121", "v122", "v123", "v124", "v125", "v126", "v127", "v128", "v129", "v130", "v131", "v132", "v133", "v134", \
              "v135", "v136", "v137", "v138", "v139", "v140", "v141", "v142", "v143", "v144", "v145", "v146", "v147", "v148", "v149", \
              "v150", "v151", "v169", "v170", "v176", "v177", "v178", "v179", "v180", "v181", "v182", "v183", "v184", "v185", "v186", \
              "v187", "v188", "v189", "v190", "v191", "s54", "s55", "scc", "vcc", "memory"
        if constexpr (std::is_same<T, f16_t>::value) asm volatile(PREFILL_LOOP_F16 PREFILL_LOOP_OPERANDS);
        else asm volatile(PREFILL_LOOP_BF16 PREFILL_LOOP_OPERANDS);
#undef PREFILL_LOOP_OPERANDS
        pf[0] = p0; pf[1] = p1;
        l_run[0] += ps0; l_run[1] += ps1;
        for (int i = 0; i < (n & 3); i++) { next_k_unit(); next_v_unit(); }
        k_unit += n & ~3; v_unit += n & ~3;
    };
    // one word per wave behind the tile memory, a set of four per (pass, attempt) parity so that no set is cleared or reused early
    uint32_t* const redo_flag = (uint32_t*)(smem + 2 * KBYTES + 4 * 32 * 272) + 4 * (pass & 1);
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
    m_ref[0] = m_ref[1] = -INFINITY; l_run[0] = l_run[1] = 0.0f;
    while (k_unit & 3) next_k_unit();           // (a second attempt starts from unit 0 again)
    while (v_unit & 3) next_v_unit();
    k_unit = 0; v_unit = 0;
    if (!safe) {
        // Q, K(0) and K(1) are on their way (open_pass); V(0) is asked for now and waited for only after S(0), P(0) and S(1): the
        // wait below leaves this wave's last four loads, which are those of V(0), outstanding (loads complete in issue order)
        if (ntiles > 0) { issue_v(V, 0); asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); }
        else __builtin_amdgcn_s_waitcnt(0);
        __syncthreads();
    } else {
        if (ntiles > 0) { issue_k(K, 0); issue_v(V, 0); }
        if (ntiles > 1) issue_k(K, 1);
        tile_barrier();
    }
    STAMP(1);
    if (nu > 0) qk_plain();                     // S(0)
    next_k_unit();                              // K addresses at unit 1, V addresses at unit 0
    // unit 0 (nothing accumulated yet): P(0), S(1), the tile barrier of an even unit
    if (nu > 0) softmax_exact(0, 0 > ufull, true);
    if (nu > 1) qk_plain();
    next_k_unit();
    tile_barrier();
    int u = 1;
    while (u < nunits) {
        if (!safe && u == 1) {
            // one run of the assembly loop: units 1 .. u_last, whole, unmasked, with a successor; it ends ahead of the odd unit
            // that would have to load a partial tile (the last tile of a sequence that is not a multiple of 64 keys long)
            const int whole = min(ntiles, Sk / BC);                 // the workgroup's tiles 0 .. whole - 1 are whole tiles
            int u_last = min(ufull, nu - 1);
            if (whole < ntiles) u_last = min(u_last, 2 * (whole - 2));      // unit 2 (whole - 2) + 1 loads tile `whole` as its K tile
            if (u_last >= 1) {
                // the unit on the causal diagonal goes with the run when it is the wave's last unit and no partial tile is about
                const bool with_diagonal = u_last == ufull && ufull + 2 == nu && whole == ntiles;
                // odd unit 2 t + 1 loads K(t + 2) for t <= whole - 3 and V(t + 1) for t <= whole - 2
                STAMP(2);
                run_units(1, u_last, max(0, whole - 2), max(0, whole - 1), with_diagonal);
                STAMP(3);
                u = u_last + 1 + (with_diagonal ? 1 : 0);
                continue;
            }
        }
        // the steps of unit u one after the other, row maxima formed first: P(u-1) V, P(u), S(u+1)
        if (u & 1) unit_loads(u);
        if (u - 1 < nu) pv_plain();
        next_v_unit();
        if (u < nu) softmax_exact(u, u > ufull, false);
        if (u + 1 < nu) qk_plain();
        next_k_unit();
        if (!(u & 1)) tile_barrier();
        u++;
    }
    if (nunits - 1 < nu && nunits > 0) pv_plain();       // P V of the workgroup's last unit
    STAMP(4);
    if (!safe) {
        const bool left_range = __builtin_amdgcn_ballot_w64(!(l_run[0] < 1.2676506e30f) || !(l_run[1] < 1.2676506e30f)) != 0ull;
        if (lane == 0) redo_flag[wave] = left_range ? 1u : 0u;
        __syncthreads();                        // the flags are written, and every wave is past its last fragment read
        const u32x4 fl = *(const u32x4*)redo_flag;
        if (__builtin_amdgcn_readfirstlane((fl[0] | fl[1] | fl[2] | fl[3])) == 0u) break;
    } else {
        __syncthreads();                        // every wave is past its last fragment read
    }
    }   // attempt

    // ---- the next pass is opened (every wave is past its last fragment read, see the end of the attempts)
    STAMP(5);
    int bh_next = 0, qt_next = 0;
    if (item + 1 < nitems) { decode(item + 1, bh_next, qt_next); open_pass(bh_next, qt_next); }
    STAMP(8);
    // ---- epilogue: normalise, store
    float l_tot[2], inv[2];
#pragma unroll
    for (int qb = 0; qb < 2; qb++) {
        l_tot[qb] = sum_over_g(l_run[qb]);
        inv[qb] = l_tot[qb] > 0.0f ? 1.0f / l_tot[qb] : 0.0f;
    }
#pragma unroll
    for (int db = 0; db < 8; db++)
#pragma unroll
        for (int qb = 0; qb < 2; qb++)
#pragma unroll
            for (int r = 0; r < 4; r++) oacc[db >> 1][4 * ((2 * db + qb) & 3) + r] *= inv[qb];
    if (a.lse && g4 == 0) {
#pragma unroll
        for (int qb = 0; qb < 2; qb++)
            if (qi[qb] < a.Sq)
                a.lse[(long long)bh * a.Sq + qi[qb]] = l_tot[qb] > 0.0f ? (m_ref[qb] + __builtin_amdgcn_logf(l_tot[qb])) * LN2 : -INFINITY;
    }
    if (Elem<OutT>::BYTES == 4 && a.vec_out) {
        // fp32 O through LDS: the lane holds 16-byte pieces of two rows (one per query block; a store instruction would touch 32 rows,
        // each a partial line); staged per wave, one half of the head dimension at a time, as [32 rows][256 B + 16] (the pad keeps
        // neighbouring rows on different banks, and leaves every LDS address a lane constant plus an immediate) in the V half of
        // the tile memory (the K half is receiving the next pass's tiles) and written back as 256-byte row halves, whole lines,
        // with non-temporal stores (O is written once and would otherwise displace K and V tiles that other workgroups re-read).
        constexpr int SROW = 272;
        unsigned char* stg = smem + 2 * KBYTES + wave_s * (32 * SROW);
        // (lane constants from an opaque copy of the lane index: they are then formed here, not ahead of the loops)
        int lnw = lane;
        asm volatile("" : "+v"(lnw));
        unsigned char* wr = stg + (lnw & 15) * SROW + (lnw >> 4) * 16;                  // piece (db % 4, g) of row 16 qb + c
        const unsigned char* rd = stg + (lnw >> 4) * SROW + (lnw & 15) * 16;           // chunk lane % 16 of row 4 q + lane / 16
        // the wave's 32 output rows: a uniform base, a 32-bit lane offset
        unsigned char* obase = (unsigned char*)((float*)a.o + ((long long)(bh * a.Sq + q0 + wave_s * 32) << 7));
        constexpr uint32_t row_bytes = 512u;
        const uint32_t lane_off = (uint32_t)(lnw >> 4) * row_bytes + (uint32_t)(lnw & 15) * 16u;
        const int rows_left = a.Sq - (q0 + wave_s * 32);                                // rows of the wave inside the sequence
#pragma unroll
        for (int half = 0; half < 2; half++) {
#pragma unroll
            for (int d4 = 0; d4 < 4; d4++)
#pragma unroll
                for (int qb = 0; qb < 2; qb++) {
                    const int db = 4 * half + d4, at = 4 * ((2 * db + qb) & 3);
                    *(f32x4*)(wr + qb * 16 * SROW + d4 * 64) = f32x4{oacc[db >> 1][at], oacc[db >> 1][at + 1], oacc[db >> 1][at + 2], oacc[db >> 1][at + 3]};
                }
            f32x4 piece[8];
#pragma unroll
            for (int q = 0; q < 8; q++) piece[q] = *(const f32x4*)(rd + 4 * q * SROW);
            if (rows_left >= 32) {
#pragma unroll
                for (int q = 0; q < 8; q++)
                    __builtin_nontemporal_store(piece[q], (f32x4*)(obase + (size_t)(4 * q) * row_bytes + 256 * half + lane_off));
            } else {
#pragma unroll
                for (int q = 0; q < 8; q++)
                    if (4 * q + (lnw >> 4) < rows_left)
                        __builtin_nontemporal_store(piece[q], (f32x4*)(obase + (size_t)(4 * q) * row_bytes + 256 * half + lane_off));
            }
#ifdef PREFILL_DBG
            if (half == 0) STAMP(9);
#endif
        }
    } else {
        typedef typename Raw2<OutT>::type out_t;
#pragma unroll
        for (int qb = 0; qb < 2; qb++) {
            if (qi[qb] >= a.Sq) continue;
            out_t* __restrict__ O = (out_t*)a.o + ((long long)(bh * a.Sq + qi[qb]) << 7);
#pragma unroll
            for (int db = 0; db < 8; db++) {
                const int d0 = 16 * db + 4 * g4, at = 4 * ((2 * db + qb) & 3);
                const float v0 = oacc[db >> 1][at], v1 = oacc[db >> 1][at + 1], v2 = oacc[db >> 1][at + 2], v3 = oacc[db >> 1][at + 3];
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
    STAMP(6);
#ifdef PREFILL_DBG
    __builtin_amdgcn_s_waitcnt(0);
    STAMP(7);
    {
        float dv = (float)(stamp[0] & 0xFFFFFFull);
#pragma unroll
        for (int i = 1; i < 8; i++) if (lane == i) dv = (float)(long long)(stamp[i] - stamp[i - 1]);
        if (lane == 8) dv = (float)(long long)(stamp[8] - stamp[5]);
        if (lane == 9) dv = (float)(long long)(stamp[9] - stamp[8]);
        if (lane == 10) dv = (float)(long long)(stamp[6] - stamp[9]);
        if (a.lse && lane < 11) a.lse[(long long)bh * a.Sq + q0 + wave_s * 32 + lane] = dv;
    }
#endif
    if (item + 1 < nitems) {
        __syncthreads();                 // the next pass's V(0) must not land on rows that are still being staged
        bh = bh_next; qt = qt_next;
    }
    }   // item
}

template <typename T, typename OutT>
static hipError_t launch_prefill(AttnArgs a, hipStream_t stream)
{
    auto kern = attn_prefill_kernel<T, OutT>;
    constexpr int smem = 2 * 64 * 256 + 4 * 32 * 272 + 64 + PREFILL_EXTRA_LDS;     // K tiles, two stages; V tiles, two stages, or the padded rows of O on their way out; the redo flags
    static unsigned long long attr_done = 0;
    if (hipError_t e = ensure_dynamic_smem((const void*)kern, smem, &attr_done)) return e;
    a.qtiles = (a.Sq + 127) / 128;
    // causal self-attention with an even number of query tiles: tile i and tile qtiles-1-i in one workgroup (equal work everywhere)
    a.paired = (a.causal && a.qoff == 0 && a.Sq == a.Sk && a.qtiles >= 2 && a.qtiles % 2 == 0) ? 1 : 0;
    const long long nblk = (long long)(a.paired ? a.qtiles / 2 : a.qtiles) * a.B * a.H;
    if (nblk > 0x7FFFFFFFLL || nblk <= 0) return hipErrorInvalidValue;
    a.nvb = (int)nblk;
    a.dgroup = make_fastdiv((uint32_t)(a.H / a.Hkv));
    a.dunits = make_fastdiv((uint32_t)(a.qtiles / 2 > 0 ? a.qtiles / 2 : 1)); a.dqtiles = make_fastdiv((uint32_t)a.qtiles);
    // two workgroups fit a CU (LDS): that many run at once, each taking its virtual blocks in turn (a multiple of the eight
    // XCDs, which the block order counts on)
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return e;
    static int cu_count[64] = {0};          // per device, asked once (benign if two threads ask at the same time: same value)
    int cus = dev >= 0 && dev < 64 ? cu_count[dev] : 0;
    if (cus == 0) {
        if (hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev)) return e;
        if (dev >= 0 && dev < 64) cu_count[dev] = cus;
    }
    const long long resident = (long long)(2 * cus) / 8 * 8;
    const unsigned grid = (unsigned)((resident >= 8 && nblk > resident) ? resident : nblk);
    a.alt_from = cus;              // workgroup b + (number of CUs) lands on the CU of workgroup b (measured: every CU of a full grid)
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), smem, stream, a);
    return hipGetLastError();
}

// The kernel takes dense [batch, head, row, 128] arrays (rows 256 bytes apart: its tile loads and its addresses count on that) whose
// row and key counts leave 32-bit index arithmetic room.
bool attn_prefill_applies(const AttnArgs& a)
{
    auto dense = [&](const long long* st, long long heads, long long rows) {
        return st[2] == 128 && (heads == 1 || st[1] == rows * 128) && (a.B == 1 || st[0] == heads * rows * 128);
    };
    if (a.D != 128 || a.nsplit > 1 || a.part || a.stream || a.bt || !(a.scale > 0.0f)) return false;
    if (a.Hkv <= 0 || a.H % a.Hkv != 0) return false;
    if (!dense(a.qs, a.H, a.Sq) || !dense(a.os, a.H, a.Sq) || !dense(a.ks, a.Hkv, a.Sk) || !dense(a.vs, a.Hkv, a.Sk)) return false;
    const long long lim = 1LL << 30;
    if (a.Sq >= lim || a.Sk >= lim || a.qoff >= lim || a.qoff <= -lim) return false;
    return (long long)a.B * a.H * a.Sq < (1LL << 31) - 256 && (long long)a.B * a.Hkv * a.Sk < (1LL << 31) - 256;
}

hipError_t launch_attn_prefill(int kind, int out16, AttnArgs a, hipStream_t stream)
{
    if (!attn_prefill_applies(a)) return hipErrorInvalidValue;
    if (kind == 1) return out16 ? launch_prefill<f16_t, f16_t>(a, stream) : launch_prefill<f16_t, float>(a, stream);
    if (kind == 2) return out16 ? launch_prefill<bf16_t, bf16_t>(a, stream) : launch_prefill<bf16_t, float>(a, stream);
    return hipErrorInvalidValue;
}

}  // namespace aidn
