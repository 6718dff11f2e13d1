#!/usr/bin/env python3
"""Writes attention_prefill_loop.inc: the run of whole, unmasked 32-key units of attn_prefill_kernel (attention_prefill.hip) as gfx950
assembly, one routine per 16-bit type.

The routine is written out by hand because the kernel's time follows what its waves issue: no moves, no address arithmetic, the
scalar work of the tile loads reduced to what the loads need, waits only where a fragment can still be outstanding.  The code is
four blocks, one per position of a unit in the two LDS stages (unit u uses block (u - 1) % 4), so every LDS offset is an
immediate; a run enters at the block of its first unit (through that block's cold start, which requests the first seven
fragments) and leaves behind any block.

Per unit u a block issues, as the C++ form of the block (full_block) does:
  slots 0..7   P(u-1) V: v_mfma into the four O accumulators; beside them FMA + exp2 of the logits of unit u (two per slot)
  slots 8..15  S(u+1) = K Q^T: v_mfma chain into the logit registers; beside them packed convert + row sum (one pair per slot)
  every slot   the LDS read of the fragment seven MFMAs ahead (ring of eight), waits counted from the reads in flight
  odd units    the direct-to-LDS loads of K(t+2), V(t+1), one per slot 0..7, while s57 / s58 say a K / V tile is left to load
  even units   the tile barrier at slot 9, behind this unit's last fragment read and ahead of the first read of the next unit

Register assignment (fixed; the kernel binds its variables to these registers at the asm statement):
  v[0:63] O accumulators, v[64:79] logits, v[80:87] P (two k-steps), v[88:119] Q fragments, v[120:151] fragment ring,
  v[152:159] K read addresses per k-step, v[160:163] V read addresses per head-dim block, v[164:167] lane offsets of the four K
  wave-loads, v168 lane offset of the V wave-loads, v169 minus the exponent reference, v170 running row sum,
  v172 v173 scratch, v[176:191] exponentials.
  s[40:41] / s[42:43] source of this wave's next K / V tile load, s44 s45 four K / V rows in bytes, s[46:47] s[48:49] one K / V
  tile in bytes, s50 s51 LDS destination of this wave's K / V loads in stage 0, s52 scale * log2(e), s53 units left,
  s[54:55] scratch, s56 block of the first unit, s57 s58 odd units that still load a K / V tile.

A second argument names parts to leave out (dma, barrier, valu, lds, vmwait): timing experiments only, the results are wrong.
"""
import os

HERE = os.path.dirname(os.path.abspath(__file__))


def gen(kind, dma=True, ablate=()):
    mfma = "v_mfma_f32_32x32x16_" + kind
    cvt = "v_cvt_pk_%s_f32" % kind
    dot = "v_dot2c_f32_%s_e32" % kind
    ones = "0x3c003c00" if kind == "f16" else "0x3f803f80"
    out = []
    emit = out.append
    queue = []          # LDS read instructions issued and not yet known complete, oldest first: fragment ids (block, index)

    def fr(j):          # ring register tuple of stream position j
        b = 120 + 4 * (j % 8)
        return b

    def read_frag(blk, f):
        """LDS reads of fragment f (0..7 V^T, 8..15 K) of block blk (0..3) into its ring slot."""
        b = fr(f)
        if "lds" in ablate:
            return
        if f < 8:
            voff = blk * 8192 + 16 * (f >> 2) * 256
            emit("ds_read_b64_tr_b16 v[%d:%d], v%d offset:%d" % (b, b + 1, 160 + (f & 3), voff))
            emit("ds_read_b64_tr_b16 v[%d:%d], v%d offset:%d" % (b + 2, b + 3, 160 + (f & 3), voff + 2048))
            queue.append((blk, f)); queue.append((blk, f))
        else:
            koff = ((blk + 2) & 3) * 8192
            emit("ds_read_b128 v[%d:%d], v%d offset:%d" % (b, b + 3, 152 + (f - 8), koff))
            queue.append((blk, f))

    def wait_frag(blk, f):
        """Wait until every read of fragment (blk, f) has returned (reads return in issue order)."""
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

    label = "L_prefill_%s_" % kind
    first7 = lambda blk: [(blk, f) for f in range(7) for _ in (0, 1)]
    # entry: s56 = phase of the first unit ((u - 1) % 4), s53 = units to run (at least one); each phase has its cold start
    for j in (1, 2, 3):
        emit("s_cmp_eq_u32 s56, %d" % j)
        emit("s_cbranch_scc1 %spre%d_%%=" % (label, j))
    for j in range(4):                      # (the compare chain above falls through into phase 0)
        emit("%spre%d_%%=:" % (label, j))
        del queue[:]
        for f in range(7):
            read_frag(j, f)
        emit("s_branch %sblk%d_%%=" % (label, j))
    for blk in range(4):
        is_b = (blk & 1) == 0               # odd units: tile loads; even units: tile barrier
        kstage = (blk >> 1) & 1             # stage of the K tile this block loads; the V tile goes to the other one
        emit("%sblk%d_%%=:" % (label, blk))
        del queue[:]
        queue.extend(first7(blk))           # what the cold start, or the block before, has left outstanding
        for i in range(16):
            if not is_b and i == 9:
                emit("s_waitcnt lgkmcnt(0)" if "vmwait" in ablate else "s_waitcnt vmcnt(0) lgkmcnt(0)")
                del queue[:]
                if "barrier" not in ablate:
                    emit("s_barrier")
            wait_frag(blk, i)
            if i < 8:
                acc = 16 * (i & 3)
                emit("%s v[%d:%d], v[%d:%d], v[%d:%d], v[%d:%d]" % (mfma, acc, acc + 15, fr(i), fr(i) + 3, 80 + 4 * (i >> 2), 83 + 4 * (i >> 2), acc, acc + 15))
            else:
                s = i - 8
                c = "0" if s == 0 else "v[64:79]"
                emit("%s v[64:79], v[%d:%d], v[%d:%d], %s" % (mfma, fr(i), fr(i) + 3, 88 + 4 * s, 91 + 4 * s, c))
            # the fragment seven MFMAs ahead
            f = i + 7
            if f < 16:
                read_frag(blk, f)
            else:
                read_frag((blk + 1) & 3, f - 16)
            if is_b and i < 8 and "dma" not in ablate:
                # this wave's share of the tile loads: K wave-loads 0..3 in slots 0..3, V wave-loads in slots 4..7; s57 / s58 count
                # the odd units that still have a K / V tile to load (vcc: whether this one has)
                k = i < 4
                n = i & 3
                ptr, step, tile, dst, lane, left = (40, 44, 46, 50, 164 + n, 57) if k else (42, 45, 48, 51, 168, 58)
                stage = kstage if k else (kstage ^ 1)
                if n == 0:
                    emit("s_cmp_lg_u32 s%d, 0" % left)
                    emit("s_cselect_b64 vcc, -1, 0")
                skip = "%sskip%d_%d_%%=" % (label, blk, i)
                emit("s_cbranch_vccz %s" % skip)
                emit("s_add_u32 m0, s%d, %d" % (dst, stage * 16384 + n * 1024))
                if n == 0:
                    emit("s_nop 0")
                    emit("global_load_lds_dwordx4 v%d, s[%d:%d]" % (lane, ptr, ptr + 1))
                else:
                    src = ptr if n == 1 else 54
                    emit("s_add_u32 s54, s%d, s%d" % (src, step))
                    emit("s_addc_u32 s55, s%d, 0" % (src + 1))
                    emit("global_load_lds_dwordx4 v%d, s[54:55]" % lane)
                if n == 3:
                    emit("s_add_u32 s%d, s%d, s%d" % (ptr, ptr, tile))
                    emit("s_addc_u32 s%d, s%d, s%d" % (ptr + 1, ptr + 1, tile + 1))
                    emit("s_sub_u32 s%d, s%d, 1" % (left, left))
                emit("%s:" % skip)
            if "valu" in ablate:
                pass
            elif i < 8:
                if i == 0:
                    emit("s_nop 3")     # the logits were written by the MFMA chain of the previous block
                emit("v_fma_f32 v172, v%d, s52, v169" % (64 + 2 * i))
                emit("v_fma_f32 v173, v%d, s52, v169" % (65 + 2 * i))
                emit("v_exp_f32_e32 v%d, v172" % (176 + 2 * i))
                emit("v_exp_f32_e32 v%d, v173" % (177 + 2 * i))
            else:
                p = i - 8
                emit("%s v%d, v%d, v%d" % (cvt, 80 + p, 176 + 2 * p, 177 + 2 * p))
                emit("%s v170, %s, v%d" % (dot, ones, 80 + p))
        assert "lds" in ablate or queue == first7((blk + 1) & 3), queue
        emit("s_sub_u32 s53, s53, 1")
        if blk < 3:
            emit("s_cmp_eq_u32 s53, 0")
            emit("s_cbranch_scc1 %sexit_%%=" % label)
        else:
            emit("s_cmp_lg_u32 s53, 0")
            emit("s_cbranch_scc1 %sblk0_%%=" % label)
    emit("%sexit_%%=:" % label)
    emit("s_waitcnt lgkmcnt(0)")
    return out


def main():
    import sys
    ablate = tuple(sys.argv[2].split(",")) if len(sys.argv) > 2 else ()
    name = sys.argv[1] if len(sys.argv) > 1 else os.path.join(HERE, "attention_prefill_loop.inc")
    with open(name, "w") as fh:
        fh.write("// Generated by gen_prefill_loop.py (the steady-state loop of attn_prefill_kernel as gfx950 assembly); do not edit.\n")
        for kind in ("f16", "bf16"):
            lines = gen(kind, True, ablate)
            fh.write("#define PREFILL_LOOP_%s \\\n" % kind.upper())
            for n, line in enumerate(lines):
                sep = "\\n" if line.endswith(":") else "\\n\\t"
                fh.write('    "%s%s"%s\n' % (line, sep, " \\" if n + 1 < len(lines) else ""))
            fh.write("// %d instructions\n" % sum(1 for x in lines if not x.endswith(":")))


if __name__ == "__main__":
    main()
