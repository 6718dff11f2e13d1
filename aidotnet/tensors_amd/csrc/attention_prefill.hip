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
    const int l32 = lane & 31, h = lane >> 5;
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
    const int nitems = (int)blockIdx.x < a.nvb ? ((a.nvb - 1 - (int)blockIdx.x) / (int)gridDim.x + 1) * npass : 0;

    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)smem);
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    const float sl2 = a.scale * LOG2E;
    const int Sk = a.Sk;
    const int qoff = a.qoff;                    // (the launcher keeps |qoff|, Sq and Sk below 2^30: row and key sums stay 32-bit)

    // Direct-to-LDS loads.  This wave's share of a tile: K wave-loads 4 w .. 4 w + 3 and the same of V, each 4 keys x 256 B; lane ->
    // (key = 4 * load + lane / 16, chunk position lane % 16).  LDS layout [key][256 B]: 16-byte chunk c of key k sits at position
    // c ^ (k & 15) in a K tile (b128 fragment reads) and at c ^ ((k & 3) << 2) in a V tile (transposing reads).
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
            for (int i = 0; i < 4; i++) attn_dma16_base(src + 4 * i * v_row_bytes, v_lane_off, dst + i * 1024);
        } else {
            int ln = lane;
            asm volatile("" : "+v"(ln));
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int key = 4 * (wave_s * 4 + i) + (ln >> 4);
                const int gkey = min(tile * BC + key, Sk - 1);
                attn_dma16(V + (long long)gkey * 128 + ((ln & 15) ^ ((key & 3) << 2)) * 8, dst + i * 1024);
            }
        }
    };
    // What opens a pass and can be asked for while the pass before it is still storing: the Q fragments (B operand of
    // S^T = K Q^T: lane (l32, h) holds row l32, elements 16 s + 8 h .. + 7) and the K tiles 0 and 1, which land in the K half of the
    // tile memory (the stores stage through the V half).
    typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));
    u32x16 qlo, qhi;                        // k-steps 0..3 and 4..7 (held the way the assembly loop takes them)
    auto qfrag = [&](int s) -> u32x4 {
        return s < 4 ? u32x4{qlo[4 * s], qlo[4 * s + 1], qlo[4 * s + 2], qlo[4 * s + 3]}
                     : u32x4{qhi[4 * s - 16], qhi[4 * s - 15], qhi[4 * s - 14], qhi[4 * s - 13]};
    };
    auto open_pass = [&](int bh, int qt) {
        int ln = lane;
        asm volatile("" : "+v"(ln));
        // (a lane whose row lies past the end of the sequence takes the last row: what it computes is never stored)
        const int qrow = min(qt * BR + wave_s * 32 + (ln & 31), a.Sq - 1);
        const uint16_t* Q = (const uint16_t*)a.q + ((long long)(bh * a.Sq) << 7) + qrow * 128 + (ln >> 5) * 8;
#pragma unroll
        for (int s = 0; s < 8; s++) {
            const u32x4 x = *(const u32x4*)(Q + 16 * s);
#pragma unroll
            for (int e = 0; e < 4; e++) { if (s < 4) qlo[4 * s + e] = x[e]; else qhi[4 * s - 16 + e] = x[e]; }
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
    const int qi = q0 + wave * 32 + l32;
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

    // ---- plain (not interleaved) forms of the three steps of a unit
    auto qk_plain = [&]() {                                    // S of the unit the K addresses point to
#pragma unroll
        for (int r = 0; r < 16; r++) sacc[r] = 0.0f;
#pragma unroll
        for (int s = 0; s < 8; s++) {
            Mma32<T>::run(sacc, k_frag(s), qfrag(s));
            if (s == 3) __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto pv_plain = [&]() {                                    // O += V^T P^T, unit the V addresses point to
#pragma unroll
        for (int s = 0; s < 8; s++) {
            Mma32<T>::run(oacc[s & 3], v_frag(s), pf[s >> 2]);
            if (s == 3) __builtin_amdgcn_sched_barrier(0);
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
    auto softmax_exact = [&](int u, bool apply_mask, const bool first) {
        if (apply_mask) mask_unit(u);
        float m = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; r++) m = fmaxf(m, sacc[r]);
        const float mloc = max_with_partner32(m) * sl2;            // scale > 0: max commutes with the scaling
        if (first) {
            m_ref = mloc < INFINITY ? mloc : -INFINITY;            // nothing accumulated yet: no O or l to move
        } else {
            // (the accumulators are scaled whether a reference moves or not, by 1 if not: a branch around the scaling costs more,
            // in copies of all 64 of them, than the scaling)
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
        // (with masked_last the run is n whole units and then unit u + n, masked first; n >= 1)
        int mask_follows = __builtin_amdgcn_readfirstlane(masked_last ? 1 : 0);
        const int mask_rel = klim - 32 * (u + n);
        const float ninf = -INFINITY;
        if (masked_last) n++;
        u32x4 p0 = pf[0], p1 = pf[1];
#define PREFILL_LOOP_OPERANDS \
            : "+{v[0:15]}"(oacc[0]), "+{v[16:31]}"(oacc[1]), "+{v[32:47]}"(oacc[2]), "+{v[48:63]}"(oacc[3]), "+{v[64:79]}"(sacc), \
              "+{v[80:83]}"(p0), "+{v[84:87]}"(p1), "+{v170}"(ps), "+{s[40:41]}"(kptr), "+{s[42:43]}"(vptr), "+{s53}"(count), "+{s57}"(kleft), "+{s58}"(vleft), "+{s59}"(mask_follows) \
            : "{v[88:103]}"(qlo), "{v[104:119]}"(qhi), "{v[152:155]}"(kad0), "{v[156:159]}"(kad1), "{v[160:163]}"(vad), \
              "{v[164:167]}"(klo), "{v168}"(vlo), "{v169}"(negm), "{s[44:51]}"(sc), "{s52}"(sl2s), "{s56}"(phase), "{v171}"(mask_rel), "{v174}"(ninf) \
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
    m_ref = -INFINITY; l_run = 0.0f;
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
        const bool left_range = __builtin_amdgcn_ballot_w64(!(l_run < 1.2676506e30f)) != 0ull;
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
    const float l_tot = sum_with_partner32(l_run);
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    if (Elem<OutT>::BYTES == 4 && a.vec_out) {
        // fp32 O through LDS: the lane holds 16-byte pieces of ONE row (64 rows per store instruction, each a partial line); staged
        // per wave, one half of the head dimension at a time, as [32 rows][256 B + 16] (the pad keeps neighbouring rows on different
        // banks, and leaves every LDS address a lane constant plus an immediate) in the V half of the tile memory (the K half is
        // receiving the next pass's tiles) and written back as 256-byte row halves, whole lines, with non-temporal stores (O is
        // written once and would otherwise displace K and V tiles that other workgroups re-read).
        constexpr int SROW = 272;
        unsigned char* stg = smem + 2 * KBYTES + wave_s * (32 * SROW);
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[i][r] *= inv;
        if (a.lse && h == 0 && qi < a.Sq)
            a.lse[(long long)bh * a.Sq + qi] = l_tot > 0.0f ? (m_ref + __builtin_amdgcn_logf(l_tot)) * LN2 : -INFINITY;
        // (lane constants from an opaque copy of the lane index: they are then formed here, not ahead of the loops)
        int lnw = lane;
        asm volatile("" : "+v"(lnw));
        unsigned char* wr = stg + (lnw & 31) * SROW + (lnw >> 5) * 16;                  // chunk 8 (i % 2) + 2 g + h of row l32
        const unsigned char* rd = stg + (lnw >> 4) * SROW + (lnw & 15) * 16;           // chunk lane % 16 of row 4 q + lane / 16
        // the wave's 32 output rows: a uniform base, a 32-bit lane offset (the launcher checks that 32 rows span less than 4 GB)
        unsigned char* obase = (unsigned char*)((float*)a.o + ((long long)(bh * a.Sq + q0 + wave_s * 32) << 7));
        constexpr uint32_t row_bytes = 512u;
        const uint32_t lane_off = (uint32_t)(lnw >> 4) * row_bytes + (uint32_t)(lnw & 15) * 16u;
        const int rows_left = a.Sq - (q0 + wave_s * 32);                                // rows of the wave inside the sequence
#pragma unroll
        for (int half = 0; half < 2; half++) {
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int g = 0; g < 4; g++)
                    *(f32x4*)(wr + (8 * i + 2 * g) * 16) = f32x4{oacc[2 * half + i][4 * g + 0], oacc[2 * half + i][4 * g + 1],
                                                                 oacc[2 * half + i][4 * g + 2], oacc[2 * half + i][4 * g + 3]};
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
    } else if (qi < a.Sq) {
        typedef typename Raw2<OutT>::type out_t;
        out_t* __restrict__ O = (out_t*)a.o + ((long long)(bh * a.Sq + qi) << 7);
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
    a.nvb = (int)nblk;
    a.dgroup = make_fastdiv((uint32_t)(a.H / a.Hkv));
    a.dunits = make_fastdiv((uint32_t)(a.qtiles / 2 > 0 ? a.qtiles / 2 : 1)); a.dqtiles = make_fastdiv((uint32_t)a.qtiles);
    const unsigned grid = (unsigned)((resident >= 8 && nblk > resident) ? resident : nblk);
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
