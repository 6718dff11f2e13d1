// Fused scaled-dot-product attention (forward) for gfx950: flash-style, one pass over K/V
// tiles streamed through LDS, QK^T and PV on MFMA, online softmax in fp32 registers.
//
// Replaces, behind the reference's GPU-backend slot, FlashAttentionV2 / FlashAttention /
// ScaledDotProductAttention (src/AiDotNet.Tensors/Engines/DirectGpu/HIP/HipBackend.cs:6118-6302,
// kernel strings Kernels/HipAttentionKernels.cs:33-232); value semantics are the CPU engine's
// (src/AiDotNet.Tensors/Engines/CpuEngine.cs:29146-29288, 27695-27881).
//
// Formulation (per workgroup: 128 query rows of one (batch, head); per wave: 32 query rows):
//   S^T = K_tile * Q^T    MFMA rows = keys, cols = queries.  Lane l then holds query (l % 32)
//                          and 16 keys per 32-key sub-tile, so the row max / sum of a query are
//                          an in-lane reduction plus ONE cross-lane exchange (lane ^ 32), and the
//                          rescale factor of the output accumulator is a per-lane scalar.
//   O^T += V_tile^T * P^T  MFMA rows = head-dim, cols = queries.  P^T in accumulator layout is
//                          already the B-operand fragment (each lane owns the keys it needs), no
//                          shuffles; V is transposed on its way into LDS ([d][key], keys of one
//                          16-group stored in fragment order so a lane's 8 keys are 16 contiguous
//                          bytes).
// K/V tiles are double-buffered in LDS: global loads of tile j+1 are issued before the MFMAs of
// tile j and stored after them, one barrier per tile.
#include "attention_common.hpp"

namespace aidn {

// DMA (fp32, plain / causal, aligned contiguous K/V): the K and V tiles go global -> LDS directly, unpadded [key][d] rows with
// XOR-swizzled 16-byte chunks (K: c ^ (key & 15) for the b128 fragment reads; V: c ^ (((key >> 2) & 1) << 3), read as the
// A operand of O^T += V^T P^T with 32-bit LDS reads, the two lane halves -- keys 4 apart -- in different bank halves).  This
// removes the register -> LDS store path (and the V transpose in registers) of the general form.
template <typename T, typename OutT, int DP, int BC, bool FULL, int MINB, bool DMA = false>
__global__ __launch_bounds__(256, MINB) void attn_fwd_kernel(const AttnArgs a)
{
    static_assert(!DMA || (!FULL && ((DP == 64 && BC == 64) || (Elem<T>::BYTES == 4 && DP == 128 && BC == 32) ||
                                     (Elem<T>::BYTES == 2 && DP == 256 && BC == 32))),
                  "DMA form: head dimension 64 with 64-key tiles (or fp32 128 / 16-bit 256 with 32-key tiles), plain / causal");
    typedef typename Raw2<T>::type raw_t;
    constexpr int E = Elem<T>::PER16, EB = Elem<T>::BYTES;
    constexpr int NT = 256, BR = 128;
    constexpr int KS = Mma32<T>::KS;
    constexpr int DSTEPS = DP / KS;            // fragment steps over the head dim (QK^T)
    constexpr int KPITCH = DP * EB + 16;       // K tile [key][d] row pitch, bytes
    constexpr int VPITCH = BC * EB + 16;       // V^T tile [d][key] row pitch, bytes
    constexpr int KBYTES = DMA ? BC * DP * EB : BC * KPITCH, VBYTES = DMA ? BC * DP * EB : DP * VPITCH;
    constexpr int KT = BC / 32;                // 32-key sub-tiles per tile
    constexpr int DT = DP / 32;                // 32-row tiles of O^T
    constexpr int PSTEPS = 32 / KS;            // PV fragment steps per key sub-tile
    constexpr int CPR = DP / E;                // 16-byte chunks per K row
    constexpr int NKC = BC * CPR;              // K chunks per tile
    constexpr int UK = (NKC + NT - 1) / NT;
    constexpr int NVU = (BC / 4) * CPR;        // V units: 4 keys x E head-dim elements
    constexpr int UV = (NVU + NT - 1) / NT;

    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char* Ks = smem;                  // [2][KBYTES]
    unsigned char* Vs = smem + 2 * KBYTES;     // [2][VBYTES]

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int l32 = lane & 31, h = lane >> 5;

    // workgroup -> (batch*head, query tile): XCD-contiguous so the q-tiles of one head share an L2;
    // late (heavy, under a causal mask) query tiles first.
    int bh, qt;
    {
        int nblk = gridDim.x, pid = blockIdx.x;
        int per = nblk >> 3, rem = nblk & 7;
        int xcd = pid & 7, idx = pid >> 3;
        int logical = (xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per) + idx;
        bh = logical / a.qtiles;
        qt = a.qtiles - 1 - (logical - bh * a.qtiles);
        if (a.causal && a.hgroup < 0) {
            // A grid that is resident all at once (at most three workgroups per CU) is not balanced by the order of
            // dispatch: hand the query tiles out heaviest first across ALL heads, so the workgroups that end up sharing a
            // CU are a heavy one and, later in the id order, a light one.
            // (the first 256 ids, one per CU, in ascending weight, so that the ids after them -- which land on the same
            // CUs in the same order -- pair the lightest of the first round with the heaviest of the second)
            const int nbh = nblk / a.qtiles;
            const int rank = (nblk > 256 && pid < 256) ? 255 - pid : pid;
            qt = a.qtiles - 1 - rank / nbh;
            bh = rank - (rank / nbh) * nbh;
        } else if (a.causal && a.hgroup > 0) {
            // A grid of several rounds: head by head (heavy tile first) leaves heavy tiles for the very end of the dispatch order
            // and a long tail (measured: a causal launch as slow as the unmasked one).  Take the heads in groups of a.hgroup and
            // hand out the query tiles of a group heaviest first across its heads, so that every group -- the last one included --
            // ends on its light tiles.  When every XCD owns whole heads the groups are formed inside the XCD's own heads.
            const bool whole = rem == 0 && per % a.qtiles == 0;
            const int heads = whole ? per / a.qtiles : nblk / a.qtiles;      // heads the groups are cut from
            const int at = whole ? idx : logical;                            // position among their workgroups
            const int gsz = heads < a.hgroup ? heads : a.hgroup;
            const int per_group = gsz * a.qtiles;
            const int grp = at / per_group, in = at - grp * per_group;
            const int first = grp * gsz;
            const int cur = heads - first < gsz ? heads - first : gsz;       // the last group may be short
            qt = a.qtiles - 1 - in / cur;
            bh = (whole ? xcd * heads : 0) + first + in % cur;
        }
    }
    const int b = bh / a.H, hd = bh - b * a.H;
    const int kvh = hd / (a.H / a.Hkv);
    const int q0 = qt * BR;
    const int qi = q0 + wave * 32 + l32;       // this lane's query row
    const bool vec = a.vec_in != 0;

    const raw_t* __restrict__ Q = (const raw_t*)a.q + b * a.qs[0] + hd * a.qs[1];
    const raw_t* __restrict__ K = (const raw_t*)a.k + b * a.ks[0] + kvh * a.ks[1];
    const raw_t* __restrict__ V = (const raw_t*)a.v + b * a.vs[0] + kvh * a.vs[1];
    const int* __restrict__ bt = a.bt ? a.bt + b * a.bt_bs : nullptr;

    // ---- Q fragments (B operand of S^T): row qi, 16-byte chunk (2 s + h).  Up to head dimension 128 they stay in registers for
    // the whole kernel; at 256 (where O alone takes 128 registers and the kernel would spill) every tile fetches them again: the
    // query tile is 128 KiB at most and stays in the CU's cache.
    constexpr bool QREG = DP <= 128;
    auto load_q = [&](int s) -> u32x4 {
        int d0 = (2 * s + h) * E;
        return (qi < a.Sq) ? ld16<T>(Q + (long long)qi * a.qs[2] + d0, a.D - d0, vec) : u32x4{0u, 0u, 0u, 0u};
    };
    u32x4 qf[QREG ? DSTEPS : 1];
    if constexpr (QREG) {
#pragma unroll
        for (int s = 0; s < DSTEPS; s++) qf[s] = load_q(s);
    }

    // ---- number of K/V tiles this query tile needs
    int ntiles = (a.Sk + BC - 1) / BC;
    if (a.causal) {
        long long lastkey = (long long)q0 + BR - 1 + a.qoff;      // largest unmasked key of the tile's last row
        if (lastkey < 0) ntiles = 0;
        else { long long nt = lastkey / BC + 1; if (nt < ntiles) ntiles = (int)nt; }
    }

    u32x4 rk[UK];
    u32x4 rv[UV * 4];

    auto load_tile = [&](int kv0) {
#pragma unroll
        for (int i = 0; i < UK; i++) {
            int u = t + i * NT;
            int row = u / CPR, ch = u - row * CPR;
            int key = kv0 + row, d0 = ch * E;
            u32x4 v = {0u, 0u, 0u, 0u};
            if ((NKC % NT == 0 || u < NKC) && key < a.Sk) v = ld16<T>(K + paged_row(bt, a.bsz, key) * a.ks[2] + d0, a.D - d0, vec);
            rk[i] = v;
        }
#pragma unroll
        for (int i = 0; i < UV; i++) {
            int u = t + i * NT;
            int kb = u % (BC / 4), db = u / (BC / 4);
            int d0 = db * E;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                int key = kv0 + kb * 4 + r;
                u32x4 v = {0u, 0u, 0u, 0u};
                if ((NVU % NT == 0 || u < NVU) && key < a.Sk) v = ld16<T>(V + paged_row(bt, a.bsz, key) * a.vs[2] + d0, a.D - d0, vec);
                rv[i * 4 + r] = v;
            }
        }
    };

    auto store_tile = [&](int stage) {
        unsigned char* ks = Ks + stage * KBYTES;
        unsigned char* vs = Vs + stage * VBYTES;
#pragma unroll
        for (int i = 0; i < UK; i++) {
            int u = t + i * NT;
            int row = u / CPR, ch = u - row * CPR;
            if (NKC % NT == 0 || u < NKC) *(u32x4*)(ks + row * KPITCH + ch * 16) = rk[i];
        }
#pragma unroll
        for (int i = 0; i < UV; i++) {
            int u = t + i * NT;
            int kb = u % (BC / 4), db = u / (BC / 4);
            if (NVU % NT == 0 || u < NVU) {
                if constexpr (E == 8) {
                    // 4 keys x 8 d  ->  8 rows (d) of 4 keys (8 bytes).  Keys of a 16-group are stored
                    // in fragment order: 4-key blocks (0,1,2,3) at block positions (0,2,1,3).
                    int blk = kb & 3;
                    int pblk = ((blk & 1) << 1) | (blk >> 1);
                    int kpos = (kb >> 2) * 16 + pblk * 4;              // in elements
#pragma unroll
                    for (int c = 0; c < 8; c++) {
                        uint32_t a0 = rv[i * 4 + 0][c >> 1], a1 = rv[i * 4 + 1][c >> 1];
                        uint32_t a2 = rv[i * 4 + 2][c >> 1], a3 = rv[i * 4 + 3][c >> 1];
                        u32x2 o;
                        if (c & 1) { o[0] = __builtin_amdgcn_perm(a1, a0, 0x07060302u); o[1] = __builtin_amdgcn_perm(a3, a2, 0x07060302u); }
                        else       { o[0] = __builtin_amdgcn_perm(a1, a0, 0x05040100u); o[1] = __builtin_amdgcn_perm(a3, a2, 0x05040100u); }
                        *(u32x2*)(vs + (db * 8 + c) * VPITCH + kpos * 2) = o;
                    }
                } else {
                    // 4 keys x 4 d -> 4 rows (d) of 4 keys (16 bytes), natural key order
#pragma unroll
                    for (int c = 0; c < 4; c++) {
                        u32x4 o = {rv[i * 4 + 0][c], rv[i * 4 + 1][c], rv[i * 4 + 2][c], rv[i * 4 + 3][c]};
                        *(u32x4*)(vs + (db * 4 + c) * VPITCH + kb * 16) = o;
                    }
                }
            }
        }
    };

    f32x16 oacc[DT];
#pragma unroll
    for (int i = 0; i < DT; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[i][r] = 0.0f;
    float m_run = -INFINITY;     // running max of the log2-domain logits of query qi (same in lanes l and l^32)
    float l_run = 0.0f;          // this lane's share of the running sum

    const int wq_min = q0 + wave * 32, wq_max = wq_min + 31;
    const float sl2 = a.scale * LOG2E;

    // DMA form: this wave's loads of a tile are K and V wave-loads 4 wave .. 4 wave + 3 (4 keys x 256 bytes each); rows past
    // the end of the sequence repeat the last key (masked below)
    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)smem);
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    // swizzles of the DMA form (chunk position of 16-byte chunk c of key row `key`):
    //   fp32 (256- / 512-byte rows): K  c ^ (key & 15);         V  c ^ (((key >> 2) & 1) << 3)   (32-bit reads, lane halves 4 keys apart)
    //   16-bit, 128-byte rows:       K  c ^ ((key >> 1) & 7);   V  c ^ (((key >> 1) & 1) << 2)   (transposing reads of 4 consecutive keys)
    //   16-bit, 512-byte rows:       K  c ^ (key & 15);         V  c ^ ((key & 3) << 2)
    constexpr bool WIDE16 = EB == 2 && DP * EB > 128;
    auto k_swz = [](int key) -> int { return (EB == 4 || WIDE16) ? (key & 15) : ((key >> 1) & 7); };
    auto v_swz = [](int key) -> int { return EB == 4 ? (((key >> 2) & 1) << 3) : WIDE16 ? ((key & 3) << 2) : (((key >> 1) & 1) << 2); };
    auto issue_tile = [&](int tile, int stage) {
        constexpr int ROWB = DP * EB;                      // 256 / 128 bytes per key row
        constexpr int KPL = 1024 / ROWB;                   // keys per 1 KiB wave-load
        constexpr int LPW = BC / KPL / 4;                  // wave-loads per wave and tile (K and V each)
        constexpr int CPRW = ROWB / 16;                    // chunks per row
        const int ld_key = lane / CPRW, ld_pos = lane % CPRW;
#pragma unroll
        for (int i = 0; i < LPW; i++) {
            const int key = KPL * (LPW * wave + i) + ld_key;               // key inside the tile
            const long long gkey = min(tile * BC + key, a.Sk - 1);
            attn_dma16(K + gkey * a.ks[2] + (ld_pos ^ k_swz(key)) * E, lds0 + stage * KBYTES + (LPW * wave_s + i) * 1024);
            attn_dma16(V + gkey * a.vs[2] + (ld_pos ^ v_swz(key)) * E,
                       lds0 + 2 * KBYTES + stage * VBYTES + (LPW * wave_s + i) * 1024);
        }
    };
    if constexpr (DMA) {
        if (ntiles > 0) issue_tile(0, 0);
        __builtin_amdgcn_s_waitcnt(0);
    } else {
        if (ntiles > 0) {
            load_tile(0);
            store_tile(0);
        }
    }
    __syncthreads();

    for (int j = 0; j < ntiles; j++) {
        const int stage = j & 1;
        const int kv0 = j * BC;
        if constexpr (DMA) { if (j + 1 < ntiles) issue_tile(j + 1, stage ^ 1); }
        else if (j + 1 < ntiles) load_tile(kv0 + BC);

        // a wave whose 32 rows are all above the causal diagonal of this tile only helps with the copies
        const bool active = !(a.causal && (long long)kv0 > (long long)wq_max + a.qoff);
        if (active) {
            const unsigned char* ks = Ks + stage * KBYTES + l32 * KPITCH + h * 16;
            const unsigned char* vs = Vs + stage * VBYTES + l32 * VPITCH + h * 16;

            f32x16 st[KT];
#pragma unroll
            for (int kt = 0; kt < KT; kt++)
#pragma unroll
                for (int r = 0; r < 16; r++) st[kt][r] = 0.0f;
            // fp32: the two MFMA phases run at a raised wave priority, ahead of the other workgroup's softmax on the SIMD (1-3 %
            // measured; the 16-bit instances lose with it)
            if constexpr (EB == 4) __builtin_amdgcn_s_setprio(2);
            constexpr int QA = 4;                 // Q fragments fetched ahead when they are not resident
            u32x4 qring[QREG ? 1 : QA];
            if constexpr (!QREG) {
#pragma unroll
                for (int s = 0; s < QA; s++) qring[s] = load_q(s);
            }
#pragma unroll
            for (int s = 0; s < DSTEPS; s++) {
                u32x4 qs;
                if constexpr (QREG) qs = qf[s];
                else {
                    qs = qring[s % QA];
                    if (s + QA < DSTEPS) qring[s % QA] = load_q(s + QA);
                }
#pragma unroll
                for (int kt = 0; kt < KT; kt++) {
                    u32x4 kf;
                    if constexpr (DMA) kf = *(const u32x4*)(Ks + stage * KBYTES + (kt * 32 + l32) * (DP * EB) + (((2 * s + h) ^ k_swz(l32)) << 4));
                    else kf = *(const u32x4*)(ks + kt * 32 * KPITCH + s * 32);
                    Mma32<T>::run(st[kt], kf, qs);
                }
            }
            if constexpr (EB == 4) __builtin_amdgcn_s_setprio(0);

            // ---- logits in the log2 domain, masks
            const bool need_mask = (kv0 + BC > a.Sk) || (a.causal && (long long)kv0 + BC - 1 > (long long)wq_min + a.qoff);
            float mloc = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < KT; kt++) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    float x;
                    const int key = kv0 + kt * 32 + acc_row(r, h);
                    if constexpr (FULL) {
                        x = st[kt][r] * a.scale;
                        if (a.softcap > 0.0f) x = a.softcap * tanhf(x / a.softcap);
                        const bool inb = qi < a.Sq && key < a.Sk;
                        if (a.bias && inb) x += a.bias[b * a.bias_bs + ((long long)hd * a.Sq + qi) * a.Sk + key];
                        if (a.mask_mode != 0 && inb) {
                            long long mi = (a.mask_mode == 2 ? ((long long)bh * a.Sq + qi) : (long long)qi) * a.Sk + key;
                            if (a.mask[mi] == 0.0f) x = -INFINITY;
                        }
                        x *= LOG2E;
                    } else {
                        x = st[kt][r] * sl2;
                    }
                    if (need_mask) {
                        if (key >= a.Sk || (a.causal && (long long)key > (long long)qi + a.qoff)) x = -INFINITY;
                    }
                    st[kt][r] = x;
                    mloc = fmaxf(mloc, x);
                }
            }
            mloc = fmaxf(mloc, shfl_xor_f(mloc, 32));
            const float m_new = fmaxf(m_run, mloc);
            const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
            m_run = m_new;

            float psum = 0.0f;
#pragma unroll
            for (int kt = 0; kt < KT; kt++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    float p = __builtin_amdgcn_exp2f(st[kt][r] - m_use);
                    st[kt][r] = p;
                    psum += p;
                }
            l_run = l_run * alpha + psum;
            // alpha == 1 in every lane (no row maximum moved) is the common case once a few tiles have been seen
            if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0ull) {
#pragma unroll
                for (int i = 0; i < DT; i++)
#pragma unroll
                    for (int r = 0; r < 16; r++) oacc[i][r] *= alpha;
            }

            // ---- O^T += V^T * P^T
            if constexpr (EB == 4) __builtin_amdgcn_s_setprio(2);
#pragma unroll
            for (int kt = 0; kt < KT; kt++) {
#pragma unroll
                for (int ps = 0; ps < PSTEPS; ps++) {
                    u32x4 pf;
                    if constexpr (E == 8) {
#pragma unroll
                        for (int w = 0; w < 4; w++) pf[w] = pack2_p<T>(st[kt][8 * ps + 2 * w], st[kt][8 * ps + 2 * w + 1]);
                    } else {
#pragma unroll
                        for (int w = 0; w < 4; w++) pf[w] = as_u32(st[kt][4 * ps + w]);
                    }
#pragma unroll
                    for (int i = 0; i < DT; i++) {
                        u32x4 vf;
                        if constexpr (DMA && EB == 4) {
                            // V[key = 32 kt + 8 ps + 4 h + q][d = 32 i + l32]; (key >> 2) & 1 == h
                            const int d = i * 32 + l32;
                            const unsigned char* vp = Vs + stage * VBYTES + (kt * 32 + 8 * ps + 4 * h) * (DP * 4) + ((((d >> 2) ^ (h << 3)) << 4) + (d & 3) * 4);
#pragma unroll
                            for (int q = 0; q < 4; q++) vf[q] = *(const uint32_t*)(vp + q * (DP * 4));
                        } else if constexpr (DMA) {
                            // 16-bit: the lane's eight k-slots are keys 16 ps + 4 h + (0..3) and 16 ps + 8 + 4 h + (0..3) (the order of
                            // the accumulator rows its P values come from); one transposing read per group of four: in a
                            // 16-lane group lane j addresses key (base + j / 4), 8 bytes at head-dim 4 (j % 4) of the 16-wide block
                            const int jl = lane & 15;
                            const int chunk = (i * 32 + 16 * ((lane >> 4) & 1) + 4 * (jl & 3)) >> 3;
#pragma unroll
                            for (int q = 0; q < 2; q++) {
                                const int row = kt * 32 + 16 * ps + 8 * q + 4 * h + (jl >> 2);
                                u32x2 w = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                    (__attribute__((address_space(3))) s16x4a*)(Vs + stage * VBYTES + row * (DP * 2) + ((chunk ^ v_swz(row)) << 4) + (jl & 1) * 8)));
                                vf[2 * q] = w[0];
                                vf[2 * q + 1] = w[1];
                            }
                        } else {
                            vf = *(const u32x4*)(vs + i * 32 * VPITCH + kt * 32 * EB + ps * 32);
                        }
                        Mma32<T>::run(oacc[i], vf, pf);
                    }
                }
            }
            if constexpr (EB == 4) __builtin_amdgcn_s_setprio(0);
        }
        if constexpr (DMA) __builtin_amdgcn_s_waitcnt(0);      // this wave's loads of tile j + 1 have landed
        else if (j + 1 < ntiles) store_tile(stage ^ 1);
        __syncthreads();
    }

    // ---- normalise and store: lane holds query qi, head-dim elements i*32 + 8 g + 4 h + (0..3)
    const float l_tot = l_run + shfl_xor_f(l_run, 32);
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    if constexpr (DMA && Elem<OutT>::BYTES == 4 && DP <= 128) {
        if (a.vec_out && a.D == DP) {
            // fp32 O through the (idle) tile memory, as in the fast kernel: staged per wave as [32 rows][DP * 4 bytes] (chunk c of row
            // r at position c ^ r) and written back as whole rows with non-temporal stores; a lane otherwise writes 16-byte pieces
            // of one row, 64 partial lines per instruction.  Every wave left the last tile at the barrier that ends the loop.
            constexpr int CH = DP / 4;                   // 16-byte chunks of a row
            constexpr int RPI = 64 / CH;                 // rows per store instruction
            unsigned char* stg = smem + wave * (32 * DP * 4);
#pragma unroll
            for (int i = 0; i < DT; i++)
#pragma unroll
                for (int g = 0; g < 4; g++)
                    *(f32x4*)(stg + l32 * (DP * 4) + (((8 * i + 2 * g + h) ^ (l32 & (CH - 1))) << 4)) =
                        f32x4{oacc[i][4 * g + 0] * inv, oacc[i][4 * g + 1] * inv, oacc[i][4 * g + 2] * inv, oacc[i][4 * g + 3] * inv};
            if (a.lse && h == 0 && qi < a.Sq)
                a.lse[(long long)bh * a.Sq + qi] = l_tot > 0.0f ? (m_run + __builtin_amdgcn_logf(l_tot)) * LN2 : -INFINITY;
            const int c = lane % CH;
#pragma unroll
            for (int q = 0; q < 32 / RPI; q++) {
                const int r = RPI * q + lane / CH;
                const int row = q0 + wave * 32 + r;
                const f32x4 v = *(const f32x4*)(stg + r * (DP * 4) + ((c ^ (r & (CH - 1))) << 4));
                f32x4* dst = (f32x4*)((float*)a.o + b * a.os[0] + hd * a.os[1] + (long long)row * a.os[2] + c * 4);
                if (row < a.Sq) __builtin_nontemporal_store(v, dst);
            }
            return;
        }
    }
    if (qi < a.Sq) {
        typedef typename Raw2<OutT>::type out_t;
        out_t* __restrict__ O = (out_t*)a.o + b * a.os[0] + hd * a.os[1] + (long long)qi * a.os[2];
#pragma unroll
        for (int i = 0; i < DT; i++) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int d0 = i * 32 + 8 * g + 4 * h;
                float v0 = oacc[i][4 * g + 0] * inv, v1 = oacc[i][4 * g + 1] * inv;
                float v2 = oacc[i][4 * g + 2] * inv, v3 = oacc[i][4 * g + 3] * inv;
                if constexpr (Elem<OutT>::BYTES == 4) {
                    if (a.vec_out && d0 + 4 <= a.D) {
                        *(f32x4*)(O + d0) = f32x4{v0, v1, v2, v3};
                    } else {
                        if (d0 + 0 < a.D) O[d0 + 0] = as_u32(v0);
                        if (d0 + 1 < a.D) O[d0 + 1] = as_u32(v1);
                        if (d0 + 2 < a.D) O[d0 + 2] = as_u32(v2);
                        if (d0 + 3 < a.D) O[d0 + 3] = as_u32(v3);
                    }
                } else {
                    uint32_t w0 = Elem<OutT>::narrow(v0) | (Elem<OutT>::narrow(v1) << 16);
                    uint32_t w1 = Elem<OutT>::narrow(v2) | (Elem<OutT>::narrow(v3) << 16);
                    if (a.vec_out && d0 + 4 <= a.D) {
                        *(u32x2*)(O + d0) = u32x2{w0, w1};
                    } else {
                        if (d0 + 0 < a.D) O[d0 + 0] = (out_t)(w0 & 0xFFFFu);
                        if (d0 + 1 < a.D) O[d0 + 1] = (out_t)(w0 >> 16);
                        if (d0 + 2 < a.D) O[d0 + 2] = (out_t)(w1 & 0xFFFFu);
                        if (d0 + 3 < a.D) O[d0 + 3] = (out_t)(w1 >> 16);
                    }
                }
            }
        }
        if (a.lse && h == 0)
            a.lse[(long long)bh * a.Sq + qi] = l_tot > 0.0f ? (m_run + __builtin_amdgcn_logf(l_tot)) * LN2 : -INFINITY;
    }
}

// ---------------------------------------------------------------------------------------------
// Fast path: 16-bit inputs, head dim 128, 16-byte aligned rows, no bias / mask / soft-cap.
// Same formulation as above (S^T = K Q^T, O^T += V^T P^T), but K and V tiles go global -> LDS with the
// gfx950 direct load (no staging registers, no ds_write, no register transposes) and V^T fragments are
// produced by the transposing LDS read:
//   K tile [64 keys][256 B]: 16-byte chunk c of key k at chunk position c ^ (k & 15)        (b128 reads)
//   V tile [64 keys][256 B]: 16-byte chunk c of key k at chunk position c ^ ((k & 3) << 2)  (tr16 reads)
// Softmax: the scale is folded into one FMA per logit (p = exp2(s * c - m)); the running max used for
// the exponent is only raised when the true max has grown by more than 8 (log2 units), so the O
// accumulator is rescaled rarely and P never exceeds 2^8 -- exact mathematics, LSE = m + log2(l) holds
// for any reference point m.


// Heads whose query tiles are interleaved (heaviest first) in the causal workgroup order of one XCD: 4 heads x 1 MiB of K and V
// (S = 2048, d = 128, 16-bit) is what one XCD's 4 MiB L2 holds, and four heads' tiles are enough to balance the CUs.
#define ATTN_HEAD_GROUP 4
// Depth of the register ring that prefetches MFMA operand fragments from LDS inside a tile; must divide 8.
#define AIDN_ATTN_RING 4
template <typename T, typename OutT, int D = 128>
__global__ __launch_bounds__(256, D == 128 ? 2 : 1) void attn_fwd_dl_kernel(const AttnArgs a)
{
    typedef uint16_t raw_t;
    static_assert(D == 128 || D == 256, "head dimension 128 (two workgroups per CU) or 256 (one)");
    constexpr int BC = 64, BR = 128;
    constexpr int ROWB = 2 * D;                     // bytes of a K or V row in a tile
    constexpr int KBYTES = BC * ROWB, VBYTES = BC * ROWB;
    constexpr int DSTEPS = D / 16, DT = D / 32;
    constexpr int CH = ROWB / 16;                   // 16-byte chunks per row
    constexpr int KPL = 1024 / ROWB;                // keys per wave-load (64 lanes x 16 bytes)
    constexpr int NL = 16 / KPL;                    // wave-loads per wave and tile (a wave loads 16 keys of K and 16 of V)

    extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int l32 = lane & 31, h = lane >> 5;
    int bh, qt, split = 0;
    {
        int nblk = gridDim.x, pid = blockIdx.x;
        int per = nblk >> 3, rem = nblk & 7;
        int xcd = pid & 7, idx = pid >> 3;
        int logical = (xcd < rem ? xcd * (per + 1) : rem * (per + 1) + (xcd - rem) * per) + idx;
        bh = logical / a.qtiles;
        qt = a.qtiles - 1 - (logical - bh * a.qtiles);
        if (a.nsplit > 1) {
            // the key ranges of a query tile are neighbours; late (heavy, under a causal mask) query tiles first
            const int per_head = a.qtiles * a.nsplit;
            bh = logical / per_head;
            const int r = logical - bh * per_head;
            qt = a.qtiles - 1 - r / a.nsplit;
            split = r % a.nsplit;
        } else if (a.paired) {
            // XCD-contiguous heads, qtiles / 2 workgroups per head: first the late (heavy) tile of the pair, then the early one
            const int units = a.qtiles >> 1;
            bh = logical / units;
            qt = a.qtiles - 1 - (logical - bh * units);
        } else if (a.causal) {
            // take the heads in groups of ATTN_HEAD_GROUP and hand out the query tiles of a group heaviest first across its heads
            // (all heads at once runs as fast but re-fetches K and V 3.3 times from beyond the L2; head by head leaves a heavy
            // tile for the very end).  When every XCD owns whole heads the groups are formed inside the XCD's own heads.
            const bool whole = rem == 0 && per % a.qtiles == 0;
            const int heads = whole ? per / a.qtiles : nblk / a.qtiles;
            const int at = whole ? idx : logical;
            const int gsz = heads < ATTN_HEAD_GROUP ? heads : ATTN_HEAD_GROUP;
            const int per_group = gsz * a.qtiles;
            const int grp = at / per_group, in = at - grp * per_group;
            const int first = grp * gsz;
            const int cur = heads - first < gsz ? heads - first : gsz;   // the last group may be short
            qt = a.qtiles - 1 - in / cur;
            bh = (whole ? xcd * heads : 0) + first + in % cur;
        }
    }
    const int npass = a.paired ? 2 : 1;
    for (int pass = 0; pass < npass; pass++) {
    if (pass == 1) qt = a.qtiles - 1 - qt;
    const int b = bh / a.H, hd = bh - b * a.H;
    const int kvh = hd / (a.H / a.Hkv);
    const int q0 = qt * BR;
    const int qi = q0 + wave * 32 + l32;

    const raw_t* __restrict__ Q = (const raw_t*)a.q + b * a.qs[0] + hd * a.qs[1];
    const raw_t* __restrict__ K = (const raw_t*)a.k + b * a.ks[0] + kvh * a.ks[1];
    const raw_t* __restrict__ V = (const raw_t*)a.v + b * a.vs[0] + kvh * a.vs[1];
    // keys this workgroup sees: all of them, or its split's range (which may be empty)
    int Sk = a.Sk;
    long long qoff = a.qoff;                 // causal: query i sees keys j <= i + qoff (j counted from the first key of the range)
    if (a.nsplit > 1) {
        const int kbeg = split * a.chunk;
        K += (long long)kbeg * a.ks[2];
        V += (long long)kbeg * a.vs[2];
        Sk = max(0, min(a.chunk, a.Sk - kbeg));
        qoff -= kbeg;
    }

    u32x4 qf[DSTEPS];
#pragma unroll
    for (int s = 0; s < DSTEPS; s++) {
        u32x4 z = {0u, 0u, 0u, 0u};
        qf[s] = (qi < a.Sq) ? *(const u32x4*)(Q + (long long)qi * a.qs[2] + (2 * s + h) * 8) : z;
    }

    int ntiles = (Sk + BC - 1) / BC;
    if (a.causal) {
        long long lastkey = (long long)q0 + BR - 1 + qoff;
        if (lastkey < 0) ntiles = 0;
        else { long long nt = lastkey / BC + 1; if (nt < ntiles) ntiles = (int)nt; }
    }

    // LDS: K ring [2][KBYTES] then V ring [2][VBYTES].  This wave's DMA per tile: NL wave-loads of K and NL of V, each KPL keys
    // x ROWB bytes (4 x 256 at head dimension 128, 2 x 512 at 256); lane -> (key = KPL * load + lane / CH, chunk position = lane % CH).
    // For a tile that lies fully inside the sequence the source address is a scalar base (tile, wave, load) plus
    // a per-lane byte offset fixed for the whole kernel, so issuing a load costs no vector arithmetic.
    const uint32_t lds0 = (uint32_t)(uintptr_t)((__attribute__((address_space(3))) void*)smem);
    const int wave_s = __builtin_amdgcn_readfirstlane(wave);
    const int ld_key = lane / CH, ld_pos = lane % CH;
    const long long k_row_bytes = a.ks[2] * 2, v_row_bytes = a.vs[2] * 2;
    // (the swizzle of a lane's chunk depends on its key inside the wave's 16: load i, lane key ld_key -> key KPL i + ld_key; for V only
    // on the key's two low bits, which at 4 keys per load are ld_key for every load and at 2 keys per load alternate with the load)
    uint32_t k_lane_off[NL], v_lane_off[2];
#pragma unroll
    for (int i = 0; i < NL; i++) k_lane_off[i] = (uint32_t)(ld_key * k_row_bytes) + ((ld_pos ^ (KPL * i + ld_key)) << 4);
#pragma unroll
    for (int i = 0; i < 2; i++) v_lane_off[i] = (uint32_t)(ld_key * v_row_bytes) + ((ld_pos ^ (((KPL * i + ld_key) & 3) << 2)) << 4);
    auto issue_k = [&](int tile) {
        const uint32_t dst = lds0 + (tile & 1) * KBYTES + wave_s * (16 * ROWB);
        if (tile * BC + BC <= Sk) {
            const unsigned char* src = (const unsigned char*)K + (long long)(tile * BC + 16 * wave_s) * k_row_bytes;
            if (a.stream) {
#pragma unroll
                for (int i = 0; i < NL; i++) attn_dma16_base_stream(src + KPL * i * k_row_bytes, k_lane_off[i], dst + i * 1024);
            } else {
#pragma unroll
                for (int i = 0; i < NL; i++) attn_dma16_base(src + KPL * i * k_row_bytes, k_lane_off[i], dst + i * 1024);
            }
        } else {
#pragma unroll
            for (int i = 0; i < NL; i++) {
                int key = KPL * (wave * NL + i) + ld_key;          // key inside the tile
                int gkey = min(tile * BC + key, Sk - 1);           // clamp: rows past the end are masked later
                attn_dma16(K + (long long)gkey * a.ks[2] + (ld_pos ^ (key & 15)) * 8, dst + i * 1024);
            }
        }
    };
    auto issue_v = [&](int tile) {
        const uint32_t dst = lds0 + 2 * KBYTES + (tile & 1) * VBYTES + wave_s * (16 * ROWB);
        if (tile * BC + BC <= Sk) {
            const unsigned char* src = (const unsigned char*)V + (long long)(tile * BC + 16 * wave_s) * v_row_bytes;
            if (a.stream) {
#pragma unroll
                for (int i = 0; i < NL; i++) attn_dma16_base_stream(src + KPL * i * v_row_bytes, v_lane_off[i & 1], dst + i * 1024);
            } else {
#pragma unroll
                for (int i = 0; i < NL; i++) attn_dma16_base(src + KPL * i * v_row_bytes, v_lane_off[i & 1], dst + i * 1024);
            }
        } else {
#pragma unroll
            for (int i = 0; i < NL; i++) {
                int key = KPL * (wave * NL + i) + ld_key;
                int gkey = min(tile * BC + key, Sk - 1);
                attn_dma16(V + (long long)gkey * a.vs[2] + (ld_pos ^ ((key & 3) << 2)) * 8, dst + i * 1024);
            }
        }
    };

    f32x16 oacc[DT];
#pragma unroll
    for (int i = 0; i < DT; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[i][r] = 0.0f;
    float m_ref = -INFINITY;     // reference point of the exponent (log2 domain); same in lanes l and l ^ 32
    float l_run = 0.0f;

    const int wq_min = q0 + wave * 32, wq_max = wq_min + 31;
    const float sl2 = a.scale * LOG2E;
    // tiles this wave computes: under a causal mask a prefix of the workgroup's tiles
    int nact = wq_min < a.Sq ? ntiles : 0;      // a wave without query rows only takes part in the loads
    if (a.causal) {
        long long lk = (long long)wq_max + qoff;
        if (lk < 0) nact = 0;
        else { long long nt = lk / BC + 1; if (nt < nact) nact = (int)nt; }
    }

    // Fragment addressing.  K (b128 reads): lane reads key l32 (+ 32 per sub-tile), chunk (2 s + h) ^ (key & 15).
    // V^T (transposing reads): in a 16-lane group lane j addresses key (base + j / 4), 8 bytes at head-dim
    // 4 (j % 4) of the 16-wide block; chunk position (c + 4 dt) ^ ((key & 3) << 2).
    const int jl = lane & 15;
    const uint32_t k_lane = l32 * ROWB + ((h ^ (l32 & 15)) << 4);
    const uint32_t v_lane = (4 * h + (jl >> 2)) * ROWB + ((16 * ((lane >> 4) & 1) + 4 * (jl & 3)) >> 3) * 16 + (jl & 1) * 8
                          + ((jl >> 2) << 6);

    // last key a query may see (sequence end and causal diagonal folded into one 32-bit bound); klim carries the
    // lane's accumulator row offset 4 h so that the per-element test is against a constant
    auto key_limit = [&](int q) -> int {
        long long lim = Sk - 1;
        if (a.causal) { long long c = (long long)q + qoff; if (c < lim) lim = c; }
        return (int)(lim < -1 ? -1 : lim);
    };
    const int klim = key_limit(qi) - 4 * h;
    const int wave_klim = __builtin_amdgcn_readfirstlane(key_limit(wq_min));

    if (ntiles > 0) { issue_k(0); issue_v(0); }
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();

    // raise the exponent reference only when a row max has moved by more than 8 (or on first use)
    auto lazy_rescale = [&](float mloc) {
        if (__builtin_amdgcn_ballot_w64(mloc > m_ref + 8.0f) != 0ull) {
            const float m_new = (mloc > m_ref + 8.0f) ? mloc : m_ref;
            const float alpha = (m_new == -INFINITY) ? 1.0f : __builtin_amdgcn_exp2f(m_ref - m_new);
            m_ref = m_new;
            l_run *= alpha;
#pragma unroll
            for (int i = 0; i < DT; i++) {
                // (head dimension 256: the accumulators live in accumulation registers, which the multiply cannot read.  The two
                // opaque statements pin them there on both sides of it, so that the copies to and from vector registers are made
                // here, on this rare path, and not once per tile on the common one.)
                if constexpr (D == 256) asm volatile("" : "+a"(oacc[i]));
#pragma unroll
                for (int r = 0; r < 16; r++) oacc[i][r] *= alpha;
                if constexpr (D == 256) asm volatile("" : "+a"(oacc[i]));
            }
        }
    };
    // p = exp2(s * c - m) of two scores, rounded and packed; the row sum accumulates the rounded values (the
    // same numbers the P V product uses) with one dot instruction per pair
    auto exp_pair = [&](float s0, float s1, float m_use, uint32_t& packed, float& sum) {
        float p0 = __builtin_amdgcn_exp2f(fmaf(s0, sl2, -m_use));
        float p1 = __builtin_amdgcn_exp2f(fmaf(s1, sl2, -m_use));
        packed = pack2_p<T>(p0, p1);
        sum = add_pair<T>(packed, sum);
    };

    // Per tile (64 keys = two 32-key sub-tiles) the work of a wave is pipelined so that the exponentials sit in
    // the shadow of the matrix pipe:   S0 = QK(sub 0) | S1 = QK(sub 1) with exp(S0) | PV(sub 0) with exp(S1) | PV(sub 1)
    // invariant per-lane read addresses; ring stage, sub-tile and key block enter as immediate offsets
    // (the swizzle occupies address bits 4-7: a step or d-block index beyond them -- bit 8, head dimension 256 -- is a plain offset)
    uint32_t k_ad[8], v_ad[4];
#pragma unroll
    for (int s = 0; s < 8; s++) k_ad[s] = (lds0 + k_lane) ^ (uint32_t)(s << 5);
#pragma unroll
    for (int i = 0; i < 4; i++) v_ad[i] = (lds0 + 2 * KBYTES + v_lane) ^ (uint32_t)(i << 6);

    auto tile_body = [&](const int j, auto stage_c) {
        constexpr int stage = decltype(stage_c)::value;
        // Loads of the next tile: when this wave computes and the next tile lies fully inside the sequence they are
        // issued one per MFMA inside the first phase below (a vector-memory instruction holds the wave's issue slot for
        // some tens of cycles; there it is covered by the running MFMA).  Otherwise all at once here.
        const bool spread = !a.stream && j < nact && j + 1 < ntiles && (j + 1) * BC + BC <= Sk;
        if (j + 1 < ntiles && !spread) { issue_k(j + 1); issue_v(j + 1); }
        if (j < nact) {
            const int kv0 = j * BC;
            const bool need_mask = kv0 + BC - 1 > wave_klim;
            const int rel_lim = klim - kv0;                   // keys of this tile with index > rel_lim are masked
            auto mask_sub = [&](int kt, f32x16& st) {
#pragma unroll
                for (int r = 0; r < 16; r++)
                    if (kt * 32 + 8 * (r >> 2) + (r & 3) > rel_lim) st[r] = -INFINITY;
            };
            auto sub_max = [&](const f32x16& st) -> float {
                float m = -INFINITY;
#pragma unroll
                for (int r = 0; r < 16; r++) m = fmaxf(m, st[r]);
                return max_with_partner32(m) * sl2;            // scale > 0: max commutes with the scaling
            };

            // Fragment addresses: the swizzle is an XOR on address bits that only the lane's chunk index occupies,
            // so one base per tile and lane serves every step (XOR with a constant, then an immediate offset).
            auto k_frag = [&](int kt, int s) -> u32x4 {
                return *(const __attribute__((address_space(3))) u32x4*)(k_ad[s & 7] + (s >> 3) * 256 + stage * KBYTES + kt * 32 * ROWB);
            };
            auto v_frag8 = [&](int kt, int s) -> u32x4 {          // s = DT * (16-key half) + head-dim block
                const uint32_t ad = v_ad[(s % DT) & 3] + ((s % DT) >> 2) * 256 + stage * VBYTES + (32 * kt + 16 * (s / DT)) * ROWB;
                u32x2 w0 = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4a*)ad));
                u32x2 w1 = __builtin_bit_cast(u32x2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4a*)(ad + 8 * ROWB)));
                return u32x4{w0[0], w0[1], w1[0], w1[1]};
            };

            // LDS fragment reads run R ahead of the MFMAs that consume them (fr[] is an R-deep ring; an idle LDS read takes
            // about 90 cycles, three MFMAs); sched_barrier pins that order and the MFMA / exp interleave.
            // ---- S0 = K[0:32] Q^T
            f32x16 s0, s1;
#pragma unroll
            for (int r = 0; r < 16; r++) { s0[r] = 0.0f; s1[r] = 0.0f; }
            constexpr int R = AIDN_ATTN_RING;       // (head dimension 256, one wave per SIMD: 2 and 4 measure the same, 8 costs registers and 5-15 %)
            static_assert(DSTEPS % R == 0 && DSTEPS == 2 * DT, "the fragment ring is indexed s % R over DSTEPS steps in every phase");
            constexpr int EV = DSTEPS / 8;          // steps per pair of exponentials (eight pairs per 32-key sub-tile)
            u32x4 fr[R];
#pragma unroll
            for (int s = 0; s < R; s++) fr[s] = k_frag(0, s);
            // the phases that issue nothing but MFMAs (this one and the last) run at a raised wave priority: the matrix pipe then
            // takes them ahead of the other wave's instructions on the SIMD, whose exponentials fill the gaps (1-2 % measured)
            __builtin_amdgcn_s_setprio(2);
            if (spread) {
                const unsigned char* ksrc = (const unsigned char*)K + (long long)((j + 1) * BC + 16 * wave_s) * k_row_bytes;
                const unsigned char* vsrc = (const unsigned char*)V + (long long)((j + 1) * BC + 16 * wave_s) * v_row_bytes;
                const uint32_t kdst = lds0 + (stage ^ 1) * KBYTES + wave_s * (16 * ROWB);
                const uint32_t vdst = lds0 + 2 * KBYTES + (stage ^ 1) * VBYTES + wave_s * (16 * ROWB);
#pragma unroll
                for (int s = 0; s < DSTEPS; s++) {
                    Mma32<T>::run(s0, fr[s % R], qf[s]);
                    fr[s % R] = s + R < DSTEPS ? k_frag(0, s + R) : k_frag(1, s + R - DSTEPS);
                    if (s < NL) attn_dma16_base(ksrc + KPL * s * k_row_bytes, k_lane_off[s], kdst + s * 1024);
                    else attn_dma16_base(vsrc + KPL * (s - NL) * v_row_bytes, v_lane_off[(s - NL) & 1], vdst + (s - NL) * 1024);
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
#pragma unroll
                for (int s = 0; s < DSTEPS; s++) {
                    Mma32<T>::run(s0, fr[s % R], qf[s]);
                    fr[s % R] = s + R < DSTEPS ? k_frag(0, s + R) : k_frag(1, s + R - DSTEPS);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
            __builtin_amdgcn_s_setprio(0);
            if (need_mask) mask_sub(0, s0);
            lazy_rescale(sub_max(s0));
            float m_use = (m_ref == -INFINITY) ? 0.0f : m_ref;

            // ---- S1 = K[32:64] Q^T interleaved with P0 = exp(S0)
            u32x4 p0f[2], p1f[2];
            float psum = 0.0f;
#pragma unroll
            for (int s = 0; s < DSTEPS; s++) {
                Mma32<T>::run(s1, fr[s % R], qf[s]);
                fr[s % R] = s + R < DSTEPS ? k_frag(1, s + R) : v_frag8(0, s + R - DSTEPS);
                if (s % EV == 0) {
                    const int e = s / EV;
                    uint32_t pk;
                    exp_pair(s0[2 * e], s0[2 * e + 1], m_use, pk, psum);
                    asm volatile("" : "+v"(pk), "+v"(psum));       // keeps the exponentials here, between the MFMAs
                    p0f[e >> 2][e & 3] = pk;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            if (need_mask) mask_sub(1, s1);
            const float mloc1 = sub_max(s1);
            // ---- O^T += V[0:32]^T P0^T interleaved with P1 = exp(S1) against the standing reference
            float psum1 = 0.0f;
#pragma unroll
            for (int s = 0; s < 2 * DT; s++) {
                Mma32<T>::run(oacc[s % DT], fr[s % R], p0f[s / DT]);
                fr[s % R] = s + R < 2 * DT ? v_frag8(0, s + R) : v_frag8(1, s + R - 2 * DT);
                if (s % EV == 0) {
                    const int e = s / EV;
                    uint32_t pk;
                    exp_pair(s1[2 * e], s1[2 * e + 1], m_use, pk, psum1);
                    asm volatile("" : "+v"(pk), "+v"(psum1));
                    p1f[e >> 2][e & 3] = pk;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            l_run += psum;
            if (__builtin_amdgcn_ballot_w64(mloc1 > m_ref + 8.0f) != 0ull) {
                // rare: the second sub-tile raises the reference.  P0 (formed against the old one) is already
                // accumulated; O and l are rescaled and P1 is formed again against the new reference (the
                // values computed above may have overflowed and are dropped).
                lazy_rescale(mloc1);
                m_use = (m_ref == -INFINITY) ? 0.0f : m_ref;
                psum1 = 0.0f;
#pragma unroll
                for (int s = 0; s < 8; s++) {
                    uint32_t pk;
                    exp_pair(s1[2 * s], s1[2 * s + 1], m_use, pk, psum1);
                    p1f[s >> 2][s & 3] = pk;
                }
            }
            l_run += psum1;

            // ---- O^T += V[32:64]^T P1^T
            __builtin_amdgcn_s_setprio(2);
#pragma unroll
            for (int s = 0; s < 2 * DT; s++) {
                Mma32<T>::run(oacc[s % DT], fr[s % R], p1f[s / DT]);
                if (s + R < 2 * DT) fr[s % R] = v_frag8(1, s + R);
            }
            __builtin_amdgcn_s_setprio(0);
        }
        __builtin_amdgcn_s_waitcnt(0);      // this wave's DMA of tile j+1 has landed ...
        __syncthreads();                    // ... everyone's has, and everyone is done with tile j
    };
    for (int j = 0; j < ntiles; j += 2) {
        tile_body(j, std::integral_constant<int, 0>{});
        if (j + 1 < ntiles) tile_body(j + 1, std::integral_constant<int, 1>{});
    }

    const float l_tot = sum_with_partner32(l_run);
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    if (a.part) {
        // grouped decode over several splits: query row qi is head hd * Sq + qi of the caller; unnormalised partial for the merge
        if (qi < a.Sq) {
            float* __restrict__ P = a.part + (((long long)bh * a.Sq + qi) * a.nsplit + split) * (D + 2);
            if (h == 0) { P[0] = m_ref; P[1] = l_tot; }
#pragma unroll
            for (int i = 0; i < DT; i++)
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const int d0 = i * 32 + 8 * g + 4 * h;
                    *(u32x2*)(P + 2 + d0) = u32x2{as_u32(oacc[i][4 * g + 0]), as_u32(oacc[i][4 * g + 1])};      // 8-byte aligned
                    *(u32x2*)(P + 4 + d0) = u32x2{as_u32(oacc[i][4 * g + 2]), as_u32(oacc[i][4 * g + 3])};
                }
        }
    } else
    if (Elem<OutT>::BYTES == 4 && a.vec_out && a.stage_out) {
        // fp32 O through LDS: the lane holds 16-byte pieces of ONE row (64 rows per store instruction, each a partial line);
        // staged per wave as [32 rows][4 D bytes] (chunk c of row r at position c ^ r, conflict-free both ways) and written back
        // as whole rows, 1024 bytes per instruction (two rows at head dimension 128, one at 256).  The tile memory is idle here:
        // every wave left the last tile at the barrier that ends the loop; the barrier below keeps the next pass's loads off the
        // staged rows.
        constexpr int OROWB = 4 * D, OCH = OROWB / 16, RPI = 64 / OCH;
        unsigned char* stg = smem + wave * (32 * OROWB);
#pragma unroll
        for (int i = 0; i < DT; i++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int c = 8 * i + 2 * g + h;
                *(f32x4*)(stg + l32 * OROWB + ((c ^ l32) << 4)) =
                    f32x4{oacc[i][4 * g + 0] * inv, oacc[i][4 * g + 1] * inv, oacc[i][4 * g + 2] * inv, oacc[i][4 * g + 3] * inv};
            }
        if (a.lse && h == 0 && qi < a.Sq)
            a.lse[(long long)bh * a.Sq + qi] = l_tot > 0.0f ? (m_ref + __builtin_amdgcn_logf(l_tot)) * LN2 : -INFINITY;
        // (the lane index is taken through an opaque copy: the row addresses below are then formed here, not ahead of the tile loop)
        int ln = lane;
        asm volatile("" : "+v"(ln));
        const int c = ln % OCH;
#pragma unroll
        for (int q = 0; q < 32 / RPI; q++) {
            const int r = RPI * q + ln / OCH;
            const int row = q0 + wave * 32 + r;
            const f32x4 v = *(const f32x4*)(stg + r * OROWB + ((c ^ r) << 4));
            f32x4* dst = (f32x4*)((float*)a.o + b * a.os[0] + hd * a.os[1] + (long long)row * a.os[2] + c * 4);
            // non-temporal: O is written once and would otherwise displace K and V tiles that other workgroups re-read
            // (alternated in one process: causal B4 H32 S2048 835 -> 879 TFLOP/s, unmasked 973 -> 999, never slower)
            if (row < a.Sq) __builtin_nontemporal_store(v, dst);
        }
        if (npass > 1) __syncthreads();
    } else
    if (qi < a.Sq) {
        typedef typename Raw2<OutT>::type out_t;
        out_t* __restrict__ O = (out_t*)a.o + b * a.os[0] + hd * a.os[1] + (long long)qi * a.os[2];
#pragma unroll
        for (int i = 0; i < DT; i++) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int d0 = i * 32 + 8 * g + 4 * h;
                float v0 = oacc[i][4 * g + 0] * inv, v1 = oacc[i][4 * g + 1] * inv;
                float v2 = oacc[i][4 * g + 2] * inv, v3 = oacc[i][4 * g + 3] * inv;
                if constexpr (Elem<OutT>::BYTES == 4) {
                    if (a.vec_out) *(f32x4*)(O + d0) = f32x4{v0, v1, v2, v3};
                    else { O[d0] = as_u32(v0); O[d0 + 1] = as_u32(v1); O[d0 + 2] = as_u32(v2); O[d0 + 3] = as_u32(v3); }
                } else {
                    uint32_t w0 = Elem<OutT>::narrow(v0) | (Elem<OutT>::narrow(v1) << 16);
                    uint32_t w1 = Elem<OutT>::narrow(v2) | (Elem<OutT>::narrow(v3) << 16);
                    if (a.vec_out) *(u32x2*)(O + d0) = u32x2{w0, w1};
                    else { O[d0] = (out_t)(w0 & 0xFFFFu); O[d0 + 1] = (out_t)(w0 >> 16); O[d0 + 2] = (out_t)(w1 & 0xFFFFu); O[d0 + 3] = (out_t)(w1 >> 16); }
                }
            }
        }
        if (a.lse && h == 0)
            a.lse[(long long)bh * a.Sq + qi] = l_tot > 0.0f ? (m_ref + __builtin_amdgcn_logf(l_tot)) * LN2 : -INFINITY;
    }
    }   // pass
}

// Merge of the key-range partials of the fast kernel (head dimension 128): one workgroup per query row; the weights of the
// ranges are formed once (first wave), the partial rows are read with their loads overlapped.  part: [row][nsplit][130].
template <typename OutT>
__global__ __launch_bounds__(128) void attn_split_merge_kernel(const AttnArgs a)
{
    __shared__ float s_w[64], s_ml[2];
    const long long row = blockIdx.x;                  // (b * H + hd) * Sq + qi
    const int bh = (int)(row / a.Sq), qi = (int)(row - (long long)bh * a.Sq);
    const int b = bh / a.H, hd = bh - b * a.H;
    const float* __restrict__ P = a.part + row * a.nsplit * 130;
    const int t = threadIdx.x;
    if (t < 64) {
        const float m = t < a.nsplit ? P[t * 130] : -INFINITY;
        const float l = t < a.nsplit ? P[t * 130 + 1] : 0.0f;
        float M = m;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) M = fmaxf(M, shfl_xor_f(M, off));
        const float w = __builtin_amdgcn_exp2f(m - ((M == -INFINITY) ? 0.0f : M));
        float L = l * w;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) L += shfl_xor_f(L, off);
        s_w[t] = w;
        if (t == 0) { s_ml[0] = M; s_ml[1] = L; }
    }
    __syncthreads();
    const float M = s_ml[0], L = s_ml[1];
    float A = 0.0f;
    int s0 = 0;
    for (; s0 + 8 <= a.nsplit; s0 += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = P[(s0 + u) * 130 + 2 + t];
#pragma unroll
        for (int u = 0; u < 8; u++) A += v[u] * s_w[s0 + u];
    }
    for (; s0 < a.nsplit; s0++) A += P[s0 * 130 + 2 + t] * s_w[s0];
    typedef typename Raw2<OutT>::type out_t;
    out_t* O = (out_t*)a.o + b * a.os[0] + hd * a.os[1] + (long long)qi * a.os[2];
    const float r = L > 0.0f ? A / L : 0.0f;
    if constexpr (Elem<OutT>::BYTES == 4) O[t] = as_u32(r);
    else O[t] = (out_t)Elem<OutT>::narrow(r);
    if (t == 0 && a.lse) a.lse[row] = L > 0.0f ? (M + __builtin_amdgcn_logf(L)) * LN2 : -INFINITY;
}

template <typename T, typename OutT, int D = 128>
static hipError_t launch_attn_dl(AttnArgs a, hipStream_t stream)
{
    auto kern = attn_fwd_dl_kernel<T, OutT, D>;
    constexpr int smem = 2 * (64 * 2 * D + 64 * 2 * D);      // K and V tiles, two stages each (64 KB; 128 KB at head dimension 256)
    static unsigned long long attr_done = 0;
    if (hipError_t e = ensure_dynamic_smem((const void*)kern, smem, &attr_done)) return e;
    a.qtiles = (a.Sq + 127) / 128;
    a.stage_out = 1;
    if (D != 128 && a.nsplit > 1) return hipErrorInvalidValue;      // (the merge pass of the key ranges is written for 128)
    if (a.nsplit > 1) {
        // few query tiles over a long key sequence: every tile's keys are cut into ranges that run side by side; a merge pass follows
        a.paired = 0;
        const long long nblk = (long long)a.qtiles * a.B * a.H * a.nsplit;
        const long long rows = (long long)a.B * a.H * a.Sq;
        if (nblk > 0x7FFFFFFFLL || rows > 0x7FFFFFFFLL) return hipErrorInvalidValue;
        hipLaunchKernelGGL(kern, dim3((unsigned)nblk), dim3(256), smem, stream, a);
        if (hipError_t e = hipGetLastError()) return e;
        hipLaunchKernelGGL((attn_split_merge_kernel<OutT>), dim3((unsigned)rows), dim3(128), 0, stream, a);
        return hipGetLastError();
    }
    // causal self-attention with an even number of query tiles: pair tile i with tile qtiles-1-i, so every workgroup has the same work
    a.paired = (a.causal && a.qoff == 0 && a.Sq == a.Sk && a.qtiles >= 2 && a.qtiles % 2 == 0) ? 1 : 0;
    long long nblk = (long long)(a.paired ? a.qtiles / 2 : a.qtiles) * a.B * a.H;
    if (nblk > 0x7FFFFFFFLL) return hipErrorInvalidValue;
    hipLaunchKernelGGL(kern, dim3((unsigned)nblk), dim3(256), smem, stream, a);
    return hipGetLastError();
}

// Grouped decode (one query row per head, H / Hkv >= 2 query heads per K/V head, 16-bit, head dimension 128, contiguous aligned
// cache): the query heads of a K/V head are the rows of one query tile of the fast kernel, so a K/V row is fetched once for the
// whole group instead of once per query head.  One workgroup per (batch, K/V head, split); with several splits the partials go
// to `part` ([B*H][nsplit][130] floats: m, l, O) for the decode merge pass, with one split the kernel writes O and LSE itself.
bool attn_group_decode_applies(int kind, const AttnParams& p)
{
    if (kind == 0 || p.D != 128 || p.Sq != 1 || p.Hkv <= 0 || p.H % p.Hkv != 0 || p.block_table || !p.allow_fast_path) return false;
    const int G = p.H / p.Hkv;
    if (G < 2 || G > 128 || !(p.scale > 0.0f)) return false;
    auto al = [](const void* ptr, long long s0, long long s1, long long s2) {
        return ((uintptr_t)ptr & 15u) == 0 && (s0 * 2) % 16 == 0 && (s1 * 2) % 16 == 0 && (s2 * 2) % 16 == 0;
    };
    if (!al(p.q, p.qs[0], p.qs[1], 0) || !al(p.k, p.ks[0], p.ks[1], p.ks[2]) || !al(p.v, p.vs[0], p.vs[1], p.vs[2])) return false;
    const int oeb = p.out16 ? 2 : 4;
    if (((uintptr_t)p.o & 15u) != 0 || (p.os[0] * oeb) % 16 != 0 || (p.os[1] * oeb) % 16 != 0) return false;
    return p.ks[2] > 0 && p.ks[2] < (1LL << 28) && p.vs[2] > 0 && p.vs[2] < (1LL << 28);
}

// sk: keys every query sees (the causal offset already applied); nsplit ranges of `chunk` keys (a multiple of 64)
hipError_t attn_group_decode(hipStream_t stream, int kind, const AttnParams& p, int sk, int nsplit, int chunk, float* part)
{
    const int G = p.H / p.Hkv;
    AttnArgs a;
    a.paired = 0; a.hgroup = 0;
    a.q = p.q; a.k = p.k; a.v = p.v; a.o = p.o; a.lse = p.lse; a.bias = nullptr; a.mask = nullptr;
    a.B = p.B; a.H = p.Hkv; a.Hkv = p.Hkv; a.Sq = G; a.Sk = sk; a.D = p.D;
    a.scale = p.scale; a.causal = 0; a.qoff = 0; a.softcap = 0.0f; a.mask_mode = 0; a.bias_bs = 0;
    a.qs[0] = p.qs[0]; a.qs[1] = p.qs[1] * G; a.qs[2] = p.qs[1];        // a query row is a query head
    a.os[0] = p.os[0]; a.os[1] = p.os[1] * G; a.os[2] = p.os[1];
    for (int i = 0; i < 3; i++) { a.ks[i] = p.ks[i]; a.vs[i] = p.vs[i]; }
    a.vec_in = 1; a.vec_out = 1;
    a.bt = nullptr; a.bsz = 0; a.bt_bs = 0;
    a.nsplit = nsplit; a.chunk = chunk; a.part = nsplit > 1 ? part : nullptr; a.stream = 1; a.stage_out = 0;
    a.qtiles = 1;
    const long long nblk = (long long)p.B * p.Hkv * nsplit;
    if (nblk > 0x7FFFFFFFLL || sk <= 0) return hipErrorInvalidValue;
    constexpr int smem = 2 * (64 * 256 + 64 * 256);
    auto go = [&](auto kern) -> hipError_t {
        static unsigned long long attr_done = 0;
        if (hipError_t e = ensure_dynamic_smem((const void*)kern, smem, &attr_done)) return e;
        hipLaunchKernelGGL(kern, dim3((unsigned)nblk), dim3(256), smem, stream, a);
        return hipGetLastError();
    };
    if (kind == 1) return p.out16 ? go(attn_fwd_dl_kernel<f16_t, f16_t>) : go(attn_fwd_dl_kernel<f16_t, float>);
    return p.out16 ? go(attn_fwd_dl_kernel<bf16_t, bf16_t>) : go(attn_fwd_dl_kernel<bf16_t, float>);
}

// Normalised probabilities P[b,h,i,j] = exp(logit - LSE[b,h,i]) for callers that ask for the
// attention-weights tensor (the optional output of ScaledDotProductAttention,
// src/AiDotNet.Tensors/Engines/DirectGpu/IDirectGpuBackend.cs:1421-1424).  Not on the hot path:
// one thread per (row, key), fp32 dot product.
template <typename T>
__global__ __launch_bounds__(256) void attn_weights_kernel(const AttnArgs a, float* __restrict__ w)
{
    typedef typename Raw2<T>::type raw_t;
    long long total = (long long)a.B * a.H * a.Sq * a.Sk;
    for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (long long)gridDim.x * blockDim.x) {
        int key = (int)(idx % a.Sk);
        long long row = idx / a.Sk;
        int qi = (int)(row % a.Sq);
        int bh = (int)(row / a.Sq);
        int b = bh / a.H, hd = bh - b * a.H;
        int kvh = hd / (a.H / a.Hkv);
        const raw_t* q = (const raw_t*)a.q + b * a.qs[0] + hd * a.qs[1] + (long long)qi * a.qs[2];
        const raw_t* k = (const raw_t*)a.k + b * a.ks[0] + kvh * a.ks[1] + (long long)key * a.ks[2];
        float s = 0.0f;
        for (int d = 0; d < a.D; d++) {
            float qv, kv;
            if constexpr (Elem<T>::BYTES == 4) { qv = as_f32(q[d]); kv = as_f32(k[d]); }
            else { qv = Elem<T>::widen(q[d]); kv = Elem<T>::widen(k[d]); }
            s += qv * kv;
        }
        float x = s * a.scale;
        if (a.softcap > 0.0f) x = a.softcap * tanhf(x / a.softcap);
        if (a.bias) x += a.bias[b * a.bias_bs + ((long long)hd * a.Sq + qi) * a.Sk + key];
        bool masked = false;
        if (a.mask_mode != 0) {
            long long mi = (a.mask_mode == 2 ? ((long long)bh * a.Sq + qi) : (long long)qi) * a.Sk + key;
            masked = a.mask[mi] == 0.0f;
        }
        if (a.causal && (long long)key > (long long)qi + a.qoff) masked = true;
        float lse = a.lse[row];
        w[idx] = (masked || lse == -INFINITY) ? 0.0f : __expf(x - lse);
    }
}

// ------------------------------------------------------------------ host side
template <typename T, typename OutT, int DP, int BC, bool FULL, int MINB, bool DMA = false>
static hipError_t launch_attn(AttnArgs a, hipStream_t stream)
{
    auto kern = attn_fwd_kernel<T, OutT, DP, BC, FULL, MINB, DMA>;
    constexpr int EB = Elem<T>::BYTES;
    constexpr int smem = DMA ? 4 * BC * DP * EB : 2 * (BC * (DP * EB + 16) + DP * (BC * EB + 16));
    static unsigned long long attr_done = 0;
    if (hipError_t e = ensure_dynamic_smem((const void*)kern, smem, &attr_done)) return e;
    a.qtiles = (a.Sq + 127) / 128;
    long long nblk = (long long)a.qtiles * a.B * a.H;
    if (nblk > 0x7FFFFFFFLL) return hipErrorInvalidValue;
    // causal order: up to 768 workgroups the balanced placement of a grid that is (nearly) resident at once (measured equal or
    // better than the grouped order up to that size); beyond, groups of at least 16 heads and at least 128 workgroups
    a.hgroup = !a.causal ? 0 : nblk <= 768 ? -1 : (a.qtiles >= 8 ? 16 : (128 + a.qtiles - 1) / a.qtiles);
    hipLaunchKernelGGL(kern, dim3((unsigned)nblk), dim3(256), smem, stream, a);
    return hipGetLastError();
}

template <typename T, typename OutT, int BC>
static hipError_t dispatch_attn_d(const AttnArgs& a, bool full, hipStream_t stream)
{
    const int D = a.D;
    if (D <= 32)  return full ? launch_attn<T, OutT, 32, BC, true, 2>(a, stream)  : launch_attn<T, OutT, 32, BC, false, 2>(a, stream);
    if (D <= 64)  return full ? launch_attn<T, OutT, 64, BC, true, 2>(a, stream)  : launch_attn<T, OutT, 64, BC, false, 2>(a, stream);
    if (D <= 128) return full ? launch_attn<T, OutT, 128, BC, true, 2>(a, stream) : launch_attn<T, OutT, 128, BC, false, 2>(a, stream);
    if (D <= 256) {
        // 16-bit, plain / causal, more than two workgroups per CU: 32-key tiles, so that two workgroups share a CU (10-30 % over
        // one workgroup of 64-key tiles; smaller grids lose with it).  The other instances spill at two workgroups per CU.
        if constexpr (Elem<T>::BYTES == 2) {
            if (!full && (long long)((a.Sq + 127) / 128) * a.B * a.H > 512) return launch_attn<T, OutT, 256, 32, false, 2>(a, stream);
        }
        return full ? launch_attn<T, OutT, 256, BC, true, 1>(a, stream) : launch_attn<T, OutT, 256, BC, false, 1>(a, stream);
    }
    return hipErrorInvalidValue;
}


static bool attn_aligned16(const void* ptr, const long long* s, int bytes)
{
    return ((uintptr_t)ptr & 15u) == 0 && (s[0] * bytes) % 16 == 0 && (s[1] * bytes) % 16 == 0 && (s[2] * bytes) % 16 == 0;
}

// the fast kernel: 16-bit, head dimension 128, aligned contiguous rows, plain (optionally causal) attention
static bool attn_dl_applies(int kind, const AttnParams& p)
{
    if (kind == 0 || p.D != 128 || !(p.scale > 0.0f) || p.block_table || !p.allow_fast_path) return false;
    if (p.bias != nullptr || (p.mask && p.mask_mode != 0) || p.softcap > 0.0f) return false;
    if (!(attn_aligned16(p.q, p.qs, 2) && attn_aligned16(p.k, p.ks, 2) && attn_aligned16(p.v, p.vs, 2))) return false;
    // the kernel addresses the K/V rows of a 4-key load group with unsigned 32-bit byte offsets
    return p.ks[2] > 0 && p.ks[2] < (1LL << 28) && p.vs[2] > 0 && p.vs[2] < (1LL << 28);
}

// Key ranges per query tile for the fast kernel (1 = none): when the query tiles alone leave most CUs idle and the key
// sequence is long (chunked prefill against a long cache, a few speculative tokens), ranges of at least 512 keys up to about two
// workgroups per CU.  *chunk = keys per range (a multiple of 64).
static int attn_dl_splits(const AttnParams& p, int* chunk)
{
    const long long base = (long long)((p.Sq + 127) / 128) * p.B * p.H;
    int sk = p.Sk;
    if (p.causal) {                              // keys nobody sees do not count
        const long long lim = (long long)p.Sq + p.qoff;
        if (lim < sk) sk = (int)(lim < 0 ? 0 : lim);
    }
    *chunk = 0;
    if (base >= 256 || sk < 1024 || p.weights) return 1;
    int ns = (int)((512 + base - 1) / base);
    if (ns > sk / 512) ns = sk / 512;
    if (ns > 32) ns = 32;
    if (ns < 2) return 1;
    int c = (sk + ns - 1) / ns;
    c = (c + 63) / 64 * 64;
    ns = (sk + c - 1) / c;
    *chunk = c;
    return ns >= 2 ? ns : 1;
}

size_t attn_fwd_workspace_bytes(int kind, const AttnParams& p)
{
    if (!attn_dl_applies(kind, p)) return 0;
    int chunk;
    const int ns = attn_dl_splits(p, &chunk);
    return ns > 1 ? (size_t)p.B * p.H * p.Sq * ns * 130 * sizeof(float) : 0;
}

// kind: 0 fp32, 1 fp16, 2 bf16
hipError_t attn_fwd(hipStream_t stream, int kind, const AttnParams& p)
{
    const bool g_attn_allow_dl = p.allow_fast_path != 0;      // 0 (test hook of the context): every shape takes the general kernel
    AttnArgs a;
    a.paired = 0;
    a.hgroup = 0;
    a.nsplit = 1; a.chunk = 0; a.part = nullptr; a.stream = 0; a.stage_out = 0;
    a.q = p.q; a.k = p.k; a.v = p.v; a.o = p.o; a.lse = p.lse; a.bias = p.bias; a.mask = p.mask;
    a.B = p.B; a.H = p.H; a.Hkv = p.Hkv; a.Sq = p.Sq; a.Sk = p.Sk; a.D = p.D;
    a.scale = p.scale; a.causal = p.causal; a.qoff = p.qoff; a.softcap = p.softcap; a.mask_mode = p.mask ? p.mask_mode : 0;
    a.bias_bs = p.bias_bs;
    for (int i = 0; i < 3; i++) { a.qs[i] = p.qs[i]; a.ks[i] = p.ks[i]; a.vs[i] = p.vs[i]; a.os[i] = p.os[i]; }
    a.qtiles = 0;
    a.bt = p.block_table; a.bsz = p.block_size; a.bt_bs = p.block_table_stride;
    if (p.block_table && p.weights) return hipErrorInvalidValue;      // the weights output does not follow a block table
    const int eb = kind == 0 ? 4 : 2, e = 16 / eb;
    const int oeb = (kind == 0 || !p.out16) ? 4 : 2;
    auto al = [](const void* ptr, const long long* s, int bytes) {
        return ((uintptr_t)ptr & 15u) == 0 && (s[0] * bytes) % 16 == 0 && (s[1] * bytes) % 16 == 0 && (s[2] * bytes) % 16 == 0;
    };
    a.vec_in = (p.D % e == 0) && al(p.q, p.qs, eb) && al(p.k, p.ks, eb) && al(p.v, p.vs, eb);
    a.vec_out = (p.D % 4 == 0) && al(p.o, p.os, oeb);
    const bool full = p.bias != nullptr || a.mask_mode != 0 || p.softcap > 0.0f;
    hipError_t err;
    // fast path: 16-bit, head dim 128, aligned rows, plain (optionally causal) attention
    // the fast kernel addresses K/V rows of a 4-key load group with unsigned 32-bit byte offsets
    const bool rows32 = p.ks[2] > 0 && p.ks[2] < (1LL << 28) && p.vs[2] > 0 && p.vs[2] < (1LL << 28);
    const bool dl = kind != 0 && !full && a.vec_in && p.D == 128 && p.scale > 0.0f && rows32 && !p.block_table && g_attn_allow_dl;
    if (dl && p.workspace && attn_dl_applies(kind, p)) {
        int chunk;
        const int ns = attn_dl_splits(p, &chunk);
        if (ns > 1 && p.workspace_bytes >= (size_t)p.B * p.H * p.Sq * ns * 130 * sizeof(float)) {
            a.nsplit = ns; a.chunk = chunk; a.part = (float*)p.workspace;
        }
    }
    // Unsplit prefill has two kernels.  The software-pipelined one is the faster (894 against 840 TFLOP/s on causal B4 H32 S2048 fp16,
    // 1035 against 983 without the mask, 312 against 292 at S 128) except where a sequence ends inside a 64-key tile and the passes
    // are short: the partial tile is then a larger share of a pass, and the pipelined kernel walks it in plain steps (509 against
    // 530 at S 1100).  allow_fast_path 2 / 3 (test hooks) pin the choice.
    bool pipelined = false;
    if (dl && a.nsplit == 1 && attn_prefill_applies(a)) {      // (dense arrays: its tile loads count on rows 256 bytes apart)
        pipelined = p.allow_fast_path == 3 || (p.allow_fast_path == 1 && (p.Sk % 64 == 0 || p.Sk >= 2048));
    }
    if (pipelined) err = launch_attn_prefill(kind, p.out16, a, stream);
    else
    if (dl) {
        if (kind == 1) err = p.out16 ? launch_attn_dl<f16_t, f16_t>(a, stream) : launch_attn_dl<f16_t, float>(a, stream);
        else err = p.out16 ? launch_attn_dl<bf16_t, bf16_t>(a, stream) : launch_attn_dl<bf16_t, float>(a, stream);
    } else
    if (kind == 0) {
        // fp32: 64-key tiles while two workgroups still fit the LDS of a CU (head dimension up to 64), else 32-key tiles
        if (p.D == 64 && !full && a.vec_in && !p.block_table && g_attn_allow_dl) err = launch_attn<float, float, 64, 64, false, 2, true>(a, stream);
        else if (p.D == 128 && !full && a.vec_in && !p.block_table && g_attn_allow_dl) err = launch_attn<float, float, 128, 32, false, 2, true>(a, stream);
        else if (p.D <= 64) err = full ? (p.D <= 32 ? launch_attn<float, float, 32, 64, true, 2>(a, stream) : launch_attn<float, float, 64, 64, true, 2>(a, stream))
                                  : (p.D <= 32 ? launch_attn<float, float, 32, 64, false, 2>(a, stream) : launch_attn<float, float, 64, 64, false, 2>(a, stream));
        else err = dispatch_attn_d<float, float, 32>(a, full, stream);
    }
    else if (p.D == 256 && !full && a.vec_in && !p.block_table && g_attn_allow_dl && rows32 && p.scale > 0.0f && p.allow_fast_path != 2) {
        // head dimension 256, plain / causal, aligned rows: the phase-structured kernel at that width (64-key tiles of 512-byte rows,
        // one workgroup per CU); allow_fast_path 2 (test hook) pins the older form below
        if (kind == 1) err = p.out16 ? launch_attn_dl<f16_t, f16_t, 256>(a, stream) : launch_attn_dl<f16_t, float, 256>(a, stream);
        else err = p.out16 ? launch_attn_dl<bf16_t, bf16_t, 256>(a, stream) : launch_attn_dl<bf16_t, float, 256>(a, stream);
    }
    else if (p.D == 256 && !full && a.vec_in && !p.block_table && g_attn_allow_dl) {
        // head dimension 256, plain / causal, aligned contiguous K/V: the direct-to-LDS form on 32-key tiles (Q streamed)
        if (kind == 1) err = p.out16 ? launch_attn<f16_t, f16_t, 256, 32, false, 2, true>(a, stream) : launch_attn<f16_t, float, 256, 32, false, 2, true>(a, stream);
        else err = p.out16 ? launch_attn<bf16_t, bf16_t, 256, 32, false, 2, true>(a, stream) : launch_attn<bf16_t, float, 256, 32, false, 2, true>(a, stream);
    }
    else if (p.D == 64 && !full && a.vec_in && !p.block_table && g_attn_allow_dl) {
        // head dimension 64, plain / causal, aligned contiguous K/V: the direct-to-LDS form of the general kernel
        if (kind == 1) err = p.out16 ? launch_attn<f16_t, f16_t, 64, 64, false, 2, true>(a, stream) : launch_attn<f16_t, float, 64, 64, false, 2, true>(a, stream);
        else err = p.out16 ? launch_attn<bf16_t, bf16_t, 64, 64, false, 2, true>(a, stream) : launch_attn<bf16_t, float, 64, 64, false, 2, true>(a, stream);
    }
    else if (kind == 1) err = p.out16 ? dispatch_attn_d<f16_t, f16_t, 64>(a, full, stream) : dispatch_attn_d<f16_t, float, 64>(a, full, stream);
    else err = p.out16 ? dispatch_attn_d<bf16_t, bf16_t, 64>(a, full, stream) : dispatch_attn_d<bf16_t, float, 64>(a, full, stream);
    if (err != hipSuccess) return err;
    if (p.weights) {
        long long total = (long long)a.B * a.H * a.Sq * a.Sk;
        unsigned grid = (unsigned)((total + 255) / 256 > 65535 ? 65535 : (total + 255) / 256);
        a.lse = p.lse;
        if (kind == 0) hipLaunchKernelGGL(attn_weights_kernel<float>, dim3(grid), dim3(256), 0, stream, a, p.weights);
        else if (kind == 1) hipLaunchKernelGGL(attn_weights_kernel<f16_t>, dim3(grid), dim3(256), 0, stream, a, p.weights);
        else hipLaunchKernelGGL(attn_weights_kernel<bf16_t>, dim3(grid), dim3(256), 0, stream, a, p.weights);
        err = hipGetLastError();
    }
    return err;
}

}  // namespace aidn
