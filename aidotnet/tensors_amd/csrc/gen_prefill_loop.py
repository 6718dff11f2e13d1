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
  every slot   the LDS read of the fragment seven MFMAs ahead (ring of eight), one wait per two MFMAs, counted from the reads in flight
  odd units    the direct-to-LDS loads of K(t+2), V(t+1), one per slot 0..7, while s57 / s58 say a K / V tile is left to load
               (K and V rows are 256 bytes apart: the four loads of a wave's share differ by an immediate offset)
  even units   the tile barrier at slot 9, behind this unit's last fragment read and ahead of the first read of the next unit

Register assignment (fixed; the kernel binds its variables to these registers at the asm statement):
  v[0:63] O accumulators, v[64:79] logits, v[80:87] P (two k-steps), v[88:119] Q fragments, v[120:151] fragment ring,
  v[152:159] K read addresses per k-step, v[160:163] V read addresses per head-dim block, v[164:167] lane offsets of the four K
  wave-loads, v168 lane offset of the V wave-loads, v169 minus the exponent reference, v170 running row sum,
  v172 v173 scratch, v[176:191] exponentials.
  s[40:41] / s[42:43] source of this wave's next K / V tile load, s44 s45 unused, s[46:47] s[48:49] one K / V tile in bytes, s50 s51 LDS destination of this wave's K / V loads in stage 0, s52 scale * log2(e), s53 units left,
  s[54:55] scratch, s56 block of the first unit, s57 s58 odd units that still load a K / V tile, s59 whether a masked unit
  follows the run (then v171 holds the lane's key limit inside that unit and v174 minus infinity).

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
    def slot(blk, i, is_b, dma):
        """Slot i of block blk: the wait for its fragments (one wait per pair of slots), the MFMA, the fragment read seven ahead, this
        wave's tile load of the slot (B blocks, when dma), the vector work."""
        if not is_b and i == 9:
            emit("s_waitcnt lgkmcnt(0)" if "vmwait" in ablate else "s_waitcnt vmcnt(0) lgkmcnt(0)")
            del queue[:]
            if "barrier" not in ablate:
                emit("s_barrier")
        if (i & 1) == 0:
            wait_frag(blk, i + 1)
        else:
            wait_frag(blk, i)               # (nothing to wait for unless the barrier slot came between)
        if i < 8:
            acc = 16 * (i & 3)
            emit("%s v[%d:%d], v[%d:%d], v[%d:%d], v[%d:%d]" % (mfma, acc, acc + 15, fr(i), fr(i) + 3, 80 + 4 * (i >> 2), 83 + 4 * (i >> 2), acc, acc + 15))
        else:
            k = i - 8
            c = "0" if k == 0 else "v[64:79]"
            emit("%s v[64:79], v[%d:%d], v[%d:%d], %s" % (mfma, fr(i), fr(i) + 3, 88 + 4 * k, 91 + 4 * k, c))
        # the fragment seven MFMAs ahead
        f = i + 7
        if f < 16:
            read_frag(blk, f)
        else:
            read_frag((blk + 1) & 3, f - 16)
        if dma and "dma" not in ablate:
            # K wave-loads 0..3 in slots 0..3, V wave-loads in slots 4..7: rows are 256 bytes apart, so wave-load n lies 1024 bytes
            # behind wave-load 0 in memory and in LDS alike, and the instruction's offset moves both addresses
            n = i & 3
            ptr, lane = (40, 164 + n) if i < 4 else (42, 168)
            emit("global_load_lds_dwordx4 v%d, s[%d:%d] offset:%d" % (lane, ptr, ptr + 1, 1024 * n))
        if "valu" in ablate:
            pass
        elif i < 8:
            if i == 0:
                emit("s_nop 3")             # the logits were written by the MFMA chain of the previous block
            emit("v_fma_f32 v172, v%d, s52, v169" % (64 + 2 * i))
            emit("v_fma_f32 v173, v%d, s52, v169" % (65 + 2 * i))
            emit("v_exp_f32_e32 v%d, v172" % (176 + 2 * i))
            emit("v_exp_f32_e32 v%d, v173" % (177 + 2 * i))
        else:
            p = i - 8
            emit("%s v%d, v%d, v%d" % (cvt, 80 + p, 176 + 2 * p, 177 + 2 * p))
            emit("%s v170, %s, v%d" % (dot, ones, 80 + p))

    for blk in range(4):
        is_b = (blk & 1) == 0               # odd units: tile loads; even units: tile barrier
        kstage = (blk >> 1) & 1             # stage of the K tile this block loads; the V tile goes to the other one
        emit("%sblk%d_%%=:" % (label, blk))
        del queue[:]
        queue.extend(first7(blk))           # what the cold start, or the block before, has left outstanding
        if is_b:
            # the tile loads come four to a group (K in slots 0..3, V in slots 4..7); a group whose tile is not to be loaded (s57 /
            # s58 count the odd units that still have a K / V tile to load) runs a copy of its slots without them
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
    # The run is through.  With s59 set, one more unit follows whose logits are masked first (the unit on the causal diagonal):
    # element r of the unit goes to -inf (v174) where its key offset 8 (r / 4) + r % 4 lies beyond the lane's limit v171.
    for blk in range(4):
        emit("%sfin%d_%%=:" % (label, blk))
        emit("s_cmp_eq_u32 s59, 0")
        emit("s_cbranch_scc1 %sexit_%%=" % label)
        emit("s_mov_b32 s59, 0")
        emit("s_mov_b32 s53, 1")
        emit("s_nop 7")                     # the last MFMA of the logit chain has to have written its registers
        emit("s_nop 7")
        for r in range(16):
            emit("v_cmp_gt_i32_e32 vcc, %d, v171" % (8 * (r >> 2) + (r & 3)))
            emit("v_cndmask_b32_e32 v%d, v%d, v174, vcc" % (64 + r, 64 + r))
        emit("s_branch %sblk%d_%%=" % (label, (blk + 1) & 3))
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
