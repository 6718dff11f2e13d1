#!/usr/bin/env python3
"""Writes attention_prefill_loop.inc: the run of whole, unmasked 32-key units of attn_prefill_kernel (attention_prefill.hip) as gfx950
assembly, one routine per 16-bit type.

The routine is written out by hand because the kernel's time follows what its waves issue: no moves, no address arithmetic, the
scalar work of the tile loads reduced to what the loads need, waits only where a fragment can still be outstanding.  The code is
four blocks, one per position of a unit in the two LDS stages (unit u uses block (u - 1) % 4), so every LDS offset is an
immediate; a run enters at the block of its first unit (through that block's cold start, which requests the first seven
fragments) and leaves behind any block; with s59 set one more unit follows the run whose logits are masked first (the unit on the
causal diagonal).

No arguments: the routine into attention_prefill_loop.inc beside this script.  FILE PARTS: the routine into FILE with the comma-
separated PARTS left out (dma, barrier, valu, lds: timing experiments only, the results are wrong).
"""
import os

HERE = os.path.dirname(os.path.abspath(__file__))


def gen(kind, ablate=(), flip=0, period=1):
    """One routine on v_mfma_f32_16x16x32.  A wave's 32 queries are two blocks of 16 (qb), a unit's 32 keys two blocks of 16 (kb),
    the head dimension eight blocks of 16 (db); every fragment read from LDS feeds two MFMAs (one per query block).  Lane (c, g) =
    (lane % 16, lane / 16) holds query c of a block and keys / dims 4 g + r of a block.  Per unit u a block has 16 slots, slot i
    consuming fragment i:
      slots 0..7   the V^T fragment of d-block i: P(u-1) V into the accumulators of both query blocks; beside them FMA + exp2 of the
                   logits of unit u (two per slot)
      slots 8..15  the K fragment (kb, ks) = ((i - 8) % 2, (i - 8) / 2): the S(u+1) chains of both query blocks; beside them packed
                   convert + row sum (one pair per slot)
      every slot   the LDS read of the fragment seven slots ahead (ring of eight), one wait per two slots, counted from the reads in flight
      odd units    the direct-to-LDS loads of K(t+2), V(t+1), one per slot 0..7, while s57 / s58 say a K / V tile is left to load
                   (K and V rows are 256 bytes apart: the four loads of a wave's share differ by an immediate offset)
      even units   the tile barrier at slot 9, behind this unit's last fragment read and ahead of the first read of the next unit

    Registers (fixed; the kernel binds its variables to them at the asm statement): v[0:63] O (block (db, qb) at 4 (2 db + qb)),
    v[64:79] logits (block (kb, qb) at 64 + 4 (2 kb + qb)), v[80:87] P (qb 0, qb 1), v[88:119] Q (block (qb, ks) at
    88 + 4 (4 qb + ks)), v[120:151] fragment ring, v[152:155] K read addresses per ks (kb by an offset), v[192:199] V read
    addresses per d-block, v[160:163] lane offsets of the four K wave-loads, v164 / v174 of the even / odd V wave-loads, v165 v166 minus the
    exponent reference of query block 0 / 1, v167 v168 their running row sums, v169 v170 scratch, v171 v172 the lane's key limit
    inside a masked unit per query block, v173 minus infinity, v[176:191] exponentials.
    s[40:41] / s[42:43] source of this wave's next K / V tile load, s[46:47] s[48:49] one K / V tile in bytes, s50 s51 LDS
    destination of this wave's K / V loads in stage 0, s52 scale * log2(e), s53 units left, s56 block of the first unit, s57 s58
    odd units that still load a K / V tile, s59 whether a masked unit follows the run, s60 the priority flavour (below).

    Wave priority: the two workgroups of a CU run this routine side by side, and a SIMD serves the older of two waves of equal
    priority first -- left alone the older workgroup gets about 63 % of the issue slots, finishes early, and the younger one runs the
    last fifth of the launch on its own.  Each unit therefore starts with s_setprio ((unit / period) % 2) ^ flip: the workgroups of
    the first and of the second half of the grid (which share the CUs) take the flavours flip = 0 and flip = 1, so that at any time
    one of the two leads and they take turns; the routine leaves at priority 0.  Measured on causal and unmasked B4 H32 S2048 and
    causal S8192: the gap between the two workgroups' finish times halves (30 -> 16 us of 148) and the launch is 0.5-2.5 % shorter
    (alternating every second unit measures the same; also keeping the younger workgroup raised outside the routine closes the gap
    to 4 us and gains nothing more: the board's power management pays a lone workgroup back in clock)."""
    mfma = "v_mfma_f32_16x16x32_" + kind
    cvt = "v_cvt_pk_%s_f32" % kind
    dot = "v_dot2c_f32_%s_e32" % kind
    ones = "0x3c003c00" if kind == "f16" else "0x3f803f80"
    out = []
    emit = out.append
    queue = []

    def fr(j):
        return 120 + 4 * (j % 8)

    def read_frag(blk, f):
        b = fr(f)
        if "lds" in ablate:
            return
        if f < 8:
            voff = blk * 8192
            emit("ds_read_b64_tr_b16 v[%d:%d], v%d offset:%d" % (b, b + 1, 192 + f, voff))
            emit("ds_read_b64_tr_b16 v[%d:%d], v%d offset:%d" % (b + 2, b + 3, 192 + f, voff + 4096))
            queue.append((blk, f)); queue.append((blk, f))
        else:
            j = f - 8
            koff = ((blk + 2) & 3) * 8192 + (j & 1) * 4096
            emit("ds_read_b128 v[%d:%d], v%d offset:%d" % (b, b + 3, 152 + (j >> 1), koff))
            queue.append((blk, f))

    def wait_frag(blk, f):
        last = -1
        for n, q in enumerate(queue):
            if q == (blk, f):
                last = n
        if last < 0:
            return
        left = len(queue) - 1 - last
        assert left <= 15
        emit("s_waitcnt lgkmcnt(%d)" % left)
        del queue[:last + 1]

    label = "L_prefill_%s%s_" % (kind, "_alt" if flip else "")
    first7 = lambda blk: [(blk, f) for f in range(7) for _ in (0, 1)]
    for j in (1, 2, 3):
        emit("s_cmp_eq_u32 s56, %d" % j)
        emit("s_cbranch_scc1 %spre%d_%%=" % (label, j))
    for j in range(4):
        emit("%spre%d_%%=:" % (label, j))
        del queue[:]
        for f in range(7):
            read_frag(j, f)
        emit("s_branch %sblk%d_%%=" % (label, j))

    def slot(blk, i, is_b, dma):
        if not is_b and i == 9:
            emit("s_waitcnt vmcnt(0) lgkmcnt(0)")
            del queue[:]
            if "barrier" not in ablate:
                emit("s_barrier")
        if (i & 1) == 0:
            wait_frag(blk, i + 1)
        else:
            wait_frag(blk, i)
        f4 = "v[%d:%d]" % (fr(i), fr(i) + 3)
        if i < 8:
            for qb in (0, 1):
                o = 4 * (2 * i + qb)
                emit("%s v[%d:%d], %s, v[%d:%d], v[%d:%d]" % (mfma, o, o + 3, f4, 80 + 4 * qb, 83 + 4 * qb, o, o + 3))
        else:
            j = i - 8
            ks, kb = j >> 1, j & 1
            for qb in (0, 1):
                sb = 64 + 4 * (2 * kb + qb)
                qv = 88 + 4 * (4 * qb + ks)
                emit("%s v[%d:%d], %s, v[%d:%d], %s" % (mfma, sb, sb + 3, f4, qv, qv + 3, "0" if ks == 0 else "v[%d:%d]" % (sb, sb + 3)))
        f = i + 7
        if f < 16:
            read_frag(blk, f)
        else:
            read_frag((blk + 1) & 3, f - 16)
        if dma and "dma" not in ablate:
            n = i & 3
            ptr, lane = (40, 160 + n) if i < 4 else (42, 174 if n & 1 else 164)
            emit("global_load_lds_dwordx4 v%d, s[%d:%d] offset:%d" % (lane, ptr, ptr + 1, 1024 * n))
        if "valu" in ablate:
            pass
        elif i < 8:
            if i == 0:
                emit("s_nop 1")
            for t in (2 * i, 2 * i + 1):
                qb = (t >> 2) & 1
                emit("v_fma_f32 v%d, v%d, s52, v%d" % (169 + (t & 1), 64 + t, 165 + qb))
            for t in (2 * i, 2 * i + 1):
                emit("v_exp_f32_e32 v%d, v%d" % (176 + t, 169 + (t & 1)))
        else:
            p = i - 8
            qb, e2 = p >> 2, p & 3
            t0 = 8 * (e2 >> 1) + 4 * qb + 2 * (e2 & 1)
            emit("%s v%d, v%d, v%d" % (cvt, 80 + 4 * qb + e2, 176 + t0, 177 + t0))
            emit("%s v%d, %s, v%d" % (dot, 167 + qb, ones, 80 + 4 * qb + e2))

    for blk in range(4):
        is_b = (blk & 1) == 0
        kstage = (blk >> 1) & 1
        emit("%sblk%d_%%=:" % (label, blk))
        if "prio" not in ablate:
            emit("s_setprio %d" % ((((blk // period) & 1) ^ flip)))
        del queue[:]
        queue.extend(first7(blk))
        if is_b:
            for group in (0, 1):
                left, ptr, tile, dst, stage = (57, 40, 46, 50, kstage) if group == 0 else (58, 42, 48, 51, kstage ^ 1)
                none = "%snone%d_%d_%%=" % (label, blk, group)
                join = "%sjoin%d_%d_%%=" % (label, blk, group)
                emit("s_cmp_eq_u32 s%d, 0" % left)
                emit("s_cbranch_scc1 %s" % none)
                before = list(queue)
                emit("s_add_u32 m0, s%d, %d" % (dst, stage * 16384))
                for i in range(4 * group, 4 * group + 4):
                    slot(blk, i, True, True)
                emit("s_add_u32 s%d, s%d, s%d" % (ptr, ptr, tile))
                emit("s_addc_u32 s%d, s%d, s%d" % (ptr + 1, ptr + 1, tile + 1))
                emit("s_sub_u32 s%d, s%d, 1" % (left, left))
                emit("s_branch %s" % join)
                after = list(queue)
                emit("%s:" % none)
                queue[:] = before
                for i in range(4 * group, 4 * group + 4):
                    slot(blk, i, True, False)
                assert queue == after
                emit("%s:" % join)
            for i in range(8, 16):
                slot(blk, i, True, False)
        else:
            for i in range(16):
                slot(blk, i, False, False)
        assert "lds" in ablate or queue == first7((blk + 1) & 3), queue
        emit("s_sub_u32 s53, s53, 1")
        emit("s_cmp_eq_u32 s53, 0")
        emit("s_cbranch_scc1 %sfin%d_%%=" % (label, blk))
        if blk == 3:
            emit("s_branch %sblk0_%%=" % label)
    for blk in range(4):
        emit("%sfin%d_%%=:" % (label, blk))
        emit("s_cmp_eq_u32 s59, 0")
        emit("s_cbranch_scc1 %sexit_%%=" % label)
        emit("s_mov_b32 s59, 0")
        emit("s_mov_b32 s53, 1")
        emit("s_nop 7")
        emit("s_nop 7")
        for t in range(16):
            kb, qb, r = t >> 3, (t >> 2) & 1, t & 3
            emit("v_cmp_gt_i32_e32 vcc, %d, v%d" % (16 * kb + r, 171 + qb))
            emit("v_cndmask_b32_e32 v%d, v%d, v173, vcc" % (64 + t, 64 + t))
        emit("s_branch %sblk%d_%%=" % (label, (blk + 1) & 3))
    emit("%sexit_%%=:" % label)
    if "prio" not in ablate:
        emit("s_setprio 0")
    emit("s_waitcnt lgkmcnt(0)")
    return out


def write(name, ablate=()):
    with open(name, "w") as fh:
        fh.write("// Generated by gen_prefill_loop.py (the run of whole units of attn_prefill_kernel as gfx950 assembly); do not edit.\n")
        period = 2 if "period2" in ablate else 1
        for kind in ("f16", "bf16"):
            # both priority flavours in one statement (s60 != 0 selects the second): one set of register bindings in the kernel
            lines = ["s_cmp_eq_u32 s60, 0", "s_cbranch_scc0 L_prefill_%s_second_%%=" % kind]
            lines += gen(kind, ablate, 0, period) + ["s_branch L_prefill_%s_end_%%=" % kind, "L_prefill_%s_second_%%=:" % kind]
            lines += gen(kind, ablate, 1, period) + ["L_prefill_%s_end_%%=:" % kind]
            fh.write("#define PREFILL_LOOP_%s \\\n" % kind.upper())
            for n, line in enumerate(lines):
                sep = "\\n" if line.endswith(":") else "\\n\\t"
                fh.write('    "%s%s"%s\n' % (line, sep, " \\" if n + 1 < len(lines) else ""))
            fh.write("// %d instructions\n" % sum(1 for x in lines if not x.endswith(":")))


def main():
    import sys
    if len(sys.argv) > 1:
        write(sys.argv[1], tuple(sys.argv[2].split(",")) if len(sys.argv) > 2 else ())
    else:
        write(os.path.join(HERE, "attention_prefill_loop.inc"))


if __name__ == "__main__":
    main()
