#!/usr/bin/env python3
"""Writes the steady-state half step of the pipelined attention loop (flash_attn.hip, FaFast::half_step) as gfx950
assembly text.

One half step = 16 MFMAs of one wave: the 8 S MFMAs of the NEXT 32 keys (K fragments from LDS, Q fragments in
registers) and the 8 PV MFMAs of the CURRENT 32 keys, whose 16 scores per lane become weights on the vector ALU on
the way (fma, exp2, row sum, pack to bf16) -- plus the maximum of the next half's scores.

Why by hand: in this instruction mix (most vector instructions use a result from one or two places back) a wave
issues a vector instruction only every 8 cycles or so (two waves on a SIMD: about 6 each; independent instructions go
at one per 4), while an MFMA 32x32x16 holds the matrix pipe for 32.  Up to four vector instructions after each MFMA are
free; a phase of vector work alone, as the compiler arranges the softmax, leaves the matrix pipe idle for its whole
length.  So every MFMA here is followed by at most four vector instructions and two LDS reads, and nothing else.

Fixed registers (the kernel binds its variables to them with register constraints):
  v[0:63]     O^T accumulators, four 32 x 32 tiles (d tile dt = v[16*dt : 16*dt+15])
  v[64:79]    score tile A      v[80:95]  score tile B   (one is `cur`: scores -> weights, in place; the other is
              `next`: written by the S MFMAs)
  v[96:127]   Q fragments of the 8 d slices
  v[128:135]  LDS addresses of this lane's K fragment per d slice (stage 0, keys 0-31)
  v[136:139]  LDS addresses of this lane's V^T fragment per d tile (stage 0, keys 0-15; + 2048: its second half)
  v140        running row sum (per lane: its share)          v141  offset of the exponent (-m * log2 e, or -inf)
  v142        out: maximum of this lane's 16 scores of `next`
  v[144:175]  K fragments (8 x 4)     v[176:207]  V fragments (2 chunks x 4 d tiles x 4)     v208  scratch
  %[c]        SGPR: scale * log2 e
  %[koff]     immediate: byte offset of the K half tile (stage * 32768 + half * 8192)
  %[voff]     immediate: byte offset of the V half tile (stage * 32768 + 16384 + half * 8192)

Head dim 64 (the second pair of macros): 4 d slices and 2 d tiles, i.e. 4 S + 4 PV MFMAs for the same vector work;
O^T in v[0:31], Q fragments in v[96:111], K addresses in v[128:131], V addresses in v[136:137], V rows 128 bytes
apart.  That half step is bound by the vector ALU: its first four slots carry ten vector instructions each.

Wait states kept by construction (the assembler does not add them inside an asm statement):
  LDS data        -> MFMA       s_waitcnt lgkmcnt(n), counted here
  vector ALU      -> MFMA read  at least two instructions in between
  exp2            -> its reader at least one instruction in between
  MFMA result     -> vector ALU read   at least four MFMAs (128 cycles) in between (the maximum of `next`); after
                                       the last MFMA of the statement 11 wait states, for whatever the compiler
                                       places behind it
"""
import os
import sys

OPTS = set(filter(None, os.environ.get("GCMI_FA_OPTS", "").split(",")))  # experiments: nolds noexp novalu nomax nowait
O, SA, SB, QF, KA, VA, L, NM, MRAW, ONES, KF, VF, TMP = 0, 64, 80, 96, 128, 136, 140, 141, 142, 143, 144, 176, 208


def gen(cur, nxt, D=128):
    """D = 128: 16 MFMAs (8 S, 8 PV) per half step.  D = 64: 4 d slices and 2 d tiles, i.e. 8 MFMAs for the same vector
    work -- that variant is bound by the vector ALU, and its slots take eight vector instructions each."""
    out = []
    emit = out.append
    lds = []  # LDS reads in issue order (names)
    NDS, NDT, ROWB = D // 16, D // 32, 2 * D
    N_MFMA = NDS + 2 * NDT  # MFMAs of the half step

    def read_k(ds):
        r = KF + 4 * ds
        emit("ds_read_b128 v[%d:%d], v%d offset:%%[koff]" % (r, r + 3, KA + ds))
        lds.append("k%d" % ds)

    def read_v(ch, dt):  # chunk ch = 16 keys = 16 rows of the V tile; the second read is 8 rows further
        r = VF + 16 * ch + 4 * dt
        emit("ds_read_b64_tr_b16 v[%d:%d], v%d offset:%%[voff]+%d" % (r, r + 1, VA + dt, ch * 16 * ROWB))
        emit("ds_read_b64_tr_b16 v[%d:%d], v%d offset:%%[voff]+%d" % (r + 2, r + 3, VA + dt, ch * 16 * ROWB + 8 * ROWB))
        lds.append("v%d%d_lo" % (ch, dt))
        lds.append("v%d%d" % (ch, dt))

    def wait_for(name):
        behind = len(lds) - 1 - lds.index(name)
        emit("s_waitcnt lgkmcnt(%d)" % min(behind, 15))

    # vector work in dependency order; every item is one instruction
    def w_fma(r):
        return "v_fma_f32 v%d, v%d, %%[c], v%d" % (cur + r, cur + r, NM)

    def w_exp(r):
        return "v_exp_f32 v%d, v%d" % (cur + r, cur + r)

    def p_cvt(j):  # pair j (scores 2j, 2j+1) -> packed register: chunk a in cur+0..3, chunk b in cur+8..11
        dst = cur + (j if j < 4 else 8 + j - 4)
        return "v_cvt_pk_bf16_f32 v%d, v%d, v%d" % (dst, cur + 2 * j, cur + 2 * j + 1)

    def w_sum(r):  # before the pair's pack overwrites the weight
        return "v_add_f32 v%d, v%d, v%d" % (L, L, cur + r)

    q = []
    for r in range(16):
        q += [w_fma(r), w_exp(r)]
        if r >= 1:
            q.append(w_sum(r - 1))
        if r >= 3 and r % 2 == 1:  # pair (r-3, r-2): exponentials and sums are done
            q.append(p_cvt((r - 3) // 2))
    q += ["s_nop 0", w_sum(15), p_cvt(7)]
    # the maximum of `next` in two chains
    mx = ["v_max3_f32 v%d, v%d, v%d, v%d" % (MRAW, nxt + 0, nxt + 1, nxt + 2),
          "v_max3_f32 v%d, v%d, v%d, v%d" % (TMP, nxt + 8, nxt + 9, nxt + 10)]
    for k in range(2):
        mx.append("v_max3_f32 v%d, v%d, v%d, v%d" % (MRAW, MRAW, nxt + 3 + 2 * k, nxt + 4 + 2 * k))
        mx.append("v_max3_f32 v%d, v%d, v%d, v%d" % (TMP, TMP, nxt + 11 + 2 * k, nxt + 12 + 2 * k))
    mx.append("v_max3_f32 v%d, v%d, v%d, v%d" % (MRAW, MRAW, nxt + 7, nxt + 15))
    mx.append("s_nop 0")
    mx.append("v_max_f32 v%d, v%d, v%d" % (MRAW, MRAW, TMP))

    # the last cvt of a chunk must be two instructions ahead of the PV MFMA that reads the packed weights: check below
    def take(n):
        got = q[:n]
        del q[:n]
        return got

    # preamble: K fragments 6 deep (all 4 at D = 64); the first scores' weights fill the wait for them
    k_ahead = min(6, NDS)
    for ds in range(k_ahead):
        read_k(ds)
    for ins in take(11):  # the first four scores
        emit(ins)
    if D == 128:
        per_slot = [4] * 12 + [0] * 4
        v_reads = {slot: ((slot - 2) // 4, (slot - 2) % 4) for slot in range(2, 10)}
        max_slots = (11, 12, 13)
    else:  # the packed weights of chunk a are due before slot 4, those of chunk b before slot 6: all done in slot 4
        per_slot = [10] * 4 + [6] + [0] * 3
        v_reads = {0: (0, 0), 1: (0, 1), 2: (1, 0), 3: (1, 1)}
        max_slots = (5, 6, 7)
    for slot in range(N_MFMA):
        if slot < NDS:
            ds = slot
            wait_for("k%d" % ds)
            s = "v[%d:%d]" % (nxt, nxt + 15)
            emit("v_mfma_f32_32x32x16_bf16 %s, v[%d:%d], v[%d:%d], %s" % (s, KF + 4 * ds, KF + 4 * ds + 3, QF + 4 * ds,
                                                                      QF + 4 * ds + 3, "0" if ds == 0 else s))
        else:
            ch, dt = (slot - NDS) // NDT, (slot - NDS) % NDT
            wait_for("v%d%d" % (ch, dt))
            acc = "v[%d:%d]" % (O + 16 * dt, O + 16 * dt + 15)
            pw = cur + 8 * ch
            emit("v_mfma_f32_32x32x16_bf16 %s, v[%d:%d], v[%d:%d], %s" % (acc, VF + 16 * ch + 4 * dt, VF + 16 * ch + 4 * dt + 3, pw,
                                                                      pw + 3, acc))
        if k_ahead + slot < NDS:
            read_k(k_ahead + slot)
        elif slot in v_reads:
            read_v(*v_reads[slot])
        for ins in take(per_slot[slot]):
            emit(ins)
        if slot in max_slots:
            for ins in mx[:2]:
                emit(ins)
            del mx[:2]
    # After the last MFMA: the rest of the maximum, then enough wait states that ANY instruction the compiler puts
    # behind this statement may touch the accumulators (it does not know that MFMAs wrote them: an 8-pass MFMA's
    # result needs 11 wait states before a vector instruction reads or overwrites it).  These issue while the last
    # MFMA still holds the matrix pipe, so they cost nothing.
    for ins in mx:
        emit(ins)
    del mx[:]
    emit("s_nop 7")
    assert not q and not mx, (q, mx)
    if OPTS:
        def keep(ins):
            if "nolds" in OPTS and ins.startswith("ds_read"):
                return False
            if ("nolds" in OPTS or "nowait" in OPTS) and ins.startswith("s_waitcnt"):
                return False
            if "noexp" in OPTS and ins.startswith("v_exp"):
                return False
            if "nomax" in OPTS and ins.startswith("v_max"):
                return False
            if "novalu" in OPTS and ins.startswith("v_") and not ins.startswith("v_mfma"):
                return False
            if "nodot" in OPTS and ins.startswith("v_dot2c"):
                return False
            if "nocvt" in OPTS and ins.startswith("v_cvt"):
                return False
            if "nofma" in OPTS and ins.startswith("v_fma"):
                return False
            return True
        out = [i for i in out if keep(i)]
        return out
    # checks of the wait states promised in the header
    def writes(ins):
        return ins.split()[1].rstrip(",") if ins.startswith("v_") and not ins.startswith("v_mfma") else None

    for i, ins in enumerate(out):
        if ins.startswith("v_mfma"):
            srcs = ins.split(",")[1:3]
            lo_hi = []
            for sreg in srcs:
                a, b = sreg.strip()[2:-1].split(":")
                lo_hi.append((int(a), int(b)))
            for back in (1, 2):
                w = writes(out[i - back]) if i - back >= 0 else None
                if w and w.startswith("v") and w[1:].isdigit():
                    n = int(w[1:])
                    assert not any(a <= n <= b for a, b in lo_hi), (ins, out[i - back])
        if ins.startswith("v_exp_f32"):
            d = ins.split()[1].rstrip(",")
            nxt_ins = out[i + 1]
            assert (" " + d + ",") not in (" " + nxt_ins.split(" ", 1)[1] + ",") or nxt_ins.startswith("v_exp"), (ins, nxt_ins)
    return out


def main():
    path = sys.argv[1]
    with open(path, "w") as f:
        f.write("// generated by gen_flash_attn_halfstep.py -- do not edit\n")
        for D, tag in ((128, "FA"), (64, "FA64")):
            for name, cur, nxt in (("CUR_B", SB, SA), ("CUR_A", SA, SB)):
                f.write("#define GCMI_%s_HALF_%s \\\n" % (tag, name))
                f.write(" \\\n".join('  "%s\\n"' % ln for ln in gen(cur, nxt, D)))
                f.write("\n\n")
        f.write("#define GCMI_FA_HALF_CLOBBERS %s\n" % ", ".join('"v%d"' % r for r in range(KF, TMP + 1)))


if __name__ == "__main__":
    main()
