#!/usr/bin/env python3
"""Writes the main loop of gemm_tile256_w4_kernel (gemm_tile256.hpp) as gfx950 assembly text.

The loop keeps 256 accumulator registers, 128 fragment registers and the LDS ring's addresses in fixed registers and
places every instruction by hand: with one wave per SIMD nothing hides a stall, and the compiler's allocator does
not hold 64 accumulator tiles plus four fragment sets without copies and spills.  The kernel's set-up (addresses,
column parameters) and its epilogue stay C++; this text is one `asm volatile` statement between them.

Register contract with the kernel (inputs in fixed registers, see the constraint list in gemm_tile256.hpp):
  v[0:3]    A: byte offset of this lane inside a k-block, per DMA instruction of the wave (4 per stage)
  v[4:7]    B: the same
  v8, v9    LDS address of this lane's A fragment in slot 0 / slot 2   (+ tile*1024 + (slot&1)*32768 as offset)
  v[10:17]  LDS address of this lane's B fragment of column tile 0..7 in slot 0
  v[18:25]  the same in slot 2
  s[40:41]  A tile: address of k-block 0 (advanced by 64 bytes per block)
  s[42:43]  B tile: address of k-block 0 (advanced by s[44:45])
  s[44:45]  bytes from one k-block of B to the next
  s46       number of k-blocks / 4 - 1 (trips of the steady loop)
  s47       LDS address of this wave's 4 KiB share of slot 0's A tile (DMA target)
  s48       int8: 0x80808080 when A is u8 (the bytes are flipped to s8 on the way into the MFMA), else 0
  s49       scratch (keeps m0)
  v26       LDS address at which this lane writes accumulator tile (0, 0) for the epilogue
  a[0:255]  out: accumulator tile (jt, it) = a[(jt*8+it)*4 : +4]
  v[32:63], v[64:95]    A fragments (8 row tiles x 4 registers) of even / odd k-blocks
  v[96:127], v[128:159] B fragments (8 column tiles) of even / odd k-blocks

One stage = one k-block of 64 bytes per row = one MFMA k-step for all 64 tiles of the wave:
  s_waitcnt vmcnt(8*BEHIND) lgkmcnt(0); s_barrier     block s+1 visible to all, slot s free, own fragments of s here
  64 MFMAs, column tile by column tile, from the registers of this block's parity; between them
    the DMA of block s+4 into slot s: 8 instructions, one every 8 MFMAs (issued back to back the four waves'
    requests queue up in the address unit and stall the waves: 8 % slower), and
    the 24 fragment reads of block s+1 into the other parity's registers, one every 2 MFMAs from the second
    MFMA on (one per MFMA: 3 % slower), so that they have all returned long before the stage ends
After the last stage the accumulators of column tiles 0-3 go to LDS for the epilogue (dump()).

Measured on MI355X, bf16 4096^3 (clock counters in the kernel): the loop issues MFMAs 93-94 % of its cycles; what
is left of the time is the clock the board settles at under this power draw (1.6-1.7 GHz; 2.3 GHz with MFMAs only).

8-bit operands with u8 activations: the A fragments of block s+1 are flipped to s8 (v_xor with 0x80808080) during
stage s, one register per MFMA from the 24th MFMA on.  The A tiles are read first, and LDS returns data in order, so
each tile's four flips sit behind a partial wait (s_waitcnt lgkmcnt(n), n = the reads issued after that tile's) that
has long been satisfied; a full wait in front of the flips (all 24 reads, the last of them just issued) stalled every
stage: 12 % more cycles than a loop without flips, now 4 %.

Experiments (measurement builds only: honoured when GCMI_W4_EXPERIMENT=1 is set as well, and then the output carries
a macro that the library's sources refuse; environment variable GCMI_W4_OPTS, comma separated):
  nodma nobar nolds noxor   leave out the DMA requests / barriers / fragment reads / byte flips (wrong products)
  nodma_a nodma_b           leave out the A tile's / the B tile's requests only (wrong products)
  nolds_a nolds_b           leave out the A / the B fragment reads only ([K,N] bf16: wrong products)
  copypar                   (with nolds) block 0's fragments in both register sets, so that every MFMA has real operands
  dmaburst rdburst          other placements of the requests and the reads (correct products)
  xorlate xor1 xor0=N       the flips behind a full wait over the last 16 MFMAs / the last 32; first flip at MFMA N
"""
import os
import sys

SLOT = 32768
DUMP_PITCH = 272  # W4_DUMP_PITCH of gemm_tile256.hpp
A_BYTES = 16384
AF = [32, 64]
BF = [96, 128]
OPTS = set(filter(None, os.environ.get("GCMI_W4_OPTS", "").split(","))) if os.environ.get("GCMI_W4_EXPERIMENT") == "1" else set()


def gen(es, tb):
    mfma = "v_mfma_f32_16x16x32_bf16" if es == 2 else "v_mfma_i32_16x16x64_i8"
    trd = "ds_read_b64_tr_b16" if es == 2 else "ds_read_b64_tr_b8"
    out = []
    emit = out.append

    def dma(slot, i):
        """instructions of DMA i (0-3: A, 4-7: B) of a stage into `slot`: (set m0, load)"""
        is_b = i >= 4
        lds = slot * SLOT + (A_BYTES if is_b else 0) + (i & 3) * 1024
        return ("s_add_u32 m0, s47, %d" % lds,
                "global_load_lds_dwordx4 v%d, s[%s]" % (i, "42:43" if is_b else "40:41"))

    def advance(which):
        if which == "a":
            return ["s_add_u32 s40, s40, 64", "s_addc_u32 s41, s41, 0"]
        return ["s_add_u32 s42, s42, s44", "s_addc_u32 s43, s43, s45"]

    def read_a(slot, it, par):
        base = 8 if slot < 2 else 9
        r = AF[par] + 4 * it
        return ["ds_read_b128 v[%d:%d], v%d offset:%d" % (r, r + 3, base, (slot & 1) * SLOT + it * 1024)]

    def read_b(slot, jt, par):
        base = (10 if slot < 2 else 18) + jt
        off = (slot & 1) * SLOT
        r = BF[par] + 4 * jt
        if tb:
            return ["ds_read_b128 v[%d:%d], v%d offset:%d" % (r, r + 3, base, off)]
        return ["%s v[%d:%d], v%d offset:%d" % (trd, r, r + 1, base, off),
                "%s v[%d:%d], v%d offset:%d" % (trd, r + 2, r + 3, base, off + 2048)]

    def all_reads(slot, par):
        """the fragment reads of one k-block in the order its MFMAs want them"""
        if "nolds" in OPTS:
            return []
        if es == 1:  # the eight A tiles first: they are the ones the byte flips wait for
            rd = []
            for it in range(8):
                rd += read_a(slot, it, par)
            for jt in range(8):
                rd += read_b(slot, jt, par)
            return rd
        rd = read_b(slot, 0, par)
        for it in range(8):
            rd += read_a(slot, it, par)
        for jt in range(1, 8):
            rd += read_b(slot, jt, par)
        if "nolds_a" in OPTS:
            rd = [r for r in rd if not r.startswith("ds_read_b128")]
        if "nolds_b" in OPTS:
            rd = [r for r in rd if r.startswith("ds_read_b128")]
        return rd

    def xor_tiles(par):
        return ["v_xor_b32 v%d, s48, v%d" % (AF[par] + k, AF[par] + k) for k in range(32)]

    def stage(slot, fill, nxt, behind, loop_tail=None):
        par = slot & 1
        if nxt:
            emit("s_waitcnt vmcnt(%d) lgkmcnt(0)" % (8 * behind))
            if "nobar" not in OPTS:
                emit("s_barrier")
        else:
            emit("s_waitcnt lgkmcnt(0)")  # the last block's fragments
        extras = [[] for _ in range(64)]
        pre = []
        pos = 0
        step = 1 if "dmaburst" in OPTS else 8  # MFMAs between two DMA requests
        if fill and "nodma" not in OPTS:
            d = [dma(slot, i) for i in range(8)]
            pre.append(d[0][0])
            for i in range(8):
                if ("nodma_a" in OPTS and i < 4) or ("nodma_b" in OPTS and i >= 4):
                    continue
                extras[i * step].append(d[i][1])
                if i < 7:
                    extras[i * step + step - 1].append(d[i + 1][0])
            pos = 8 if step == 1 else 1
        if fill and "dmasame" not in OPTS:
            extras[7 * step + 1] += advance("a")
            extras[7 * step + 2] += advance("b")
        if nxt:
            rd = all_reads((slot + 1) % 4, par ^ 1)
            rstep = 1 if "rdburst" in OPTS else 2
            for k, ins in enumerate(rd):
                extras[pos + k * rstep].append(ins)
            if es == 1 and "noxor" not in OPTS:
                # u8 activations: flip the A tiles of the next block once they are here, each long before its first use
                if "xorlate" not in OPTS and "xor1" not in OPTS:
                    # LDS returns data in order: tile `it` has arrived once at most the reads issued
                    # after it are outstanding.  Flip tile by tile, four registers behind one partial wait each,
                    # one register per MFMA, starting XOR0 MFMAs into the stage.
                    xor0 = int(next((o[5:] for o in OPTS if o.startswith('xor0=')), 24))
                    x = xor_tiles(par ^ 1)
                    for it in range(8):
                        at = xor0 + 4 * it
                        issued = sum(1 for k in range(len(rd)) if pos + k * rstep <= at)  # reads issued up to here
                        dmas = min(8, at // step + 1) if fill else 0  # requests issued up to here, should they count
                        extras[at].append("s_waitcnt lgkmcnt(%d)" % max(0, min(15, issued - (it + 1) - dmas)))
                        for r in range(4):
                            extras[at + r].append(x[4 * it + r])
                elif "xor1" in OPTS:  # one register per MFMA over the second half of the stage
                    extras[31].append("s_waitcnt lgkmcnt(%d)" % (len(rd) - 9 if "rdburst" in OPTS else 0))
                    for k, ins in enumerate(xor_tiles(par ^ 1)):
                        extras[32 + k].append(ins)
                else:
                    extras[47].append("s_waitcnt lgkmcnt(0)")
                    for k, ins in enumerate(xor_tiles(par ^ 1)):
                        extras[48 + k // 2].append(ins)
        if loop_tail:
            extras[60].append("s_sub_u32 s46, s46, 1")
            extras[61].append("s_cmp_lg_u32 s46, 0")
        for ins in pre:
            emit(ins)
        for jt in range(8):
            breg = BF[par] + 4 * jt
            for it in range(8):
                acc = (jt * 8 + it) * 4
                areg = AF[par] + 4 * it
                emit("%s a[%d:%d], v[%d:%d], v[%d:%d], a[%d:%d]" % (mfma, acc, acc + 3, breg, breg + 3, areg, areg + 3,
                                                                   acc, acc + 3))
                for ins in extras[jt * 8 + it]:
                    emit(ins)
        if loop_tail:
            emit("s_cbranch_scc1 %s" % loop_tail)

    emit("s_mov_b32 s49, m0")  # m0 carries the DMA's LDS address in here; the compiler's value is put back
    # prologue: request k-blocks 0..3, clear the accumulators while they fly, take block 0 into registers
    for d in range(4):
        for i in range(8):
            m0, ld = dma(d, i)
            emit(m0)
            emit("s_nop 0")
            emit(ld)
        for ins in advance("a") + advance("b"):
            emit(ins)
    for r in range(256):
        emit("v_accvgpr_write_b32 a%d, 0" % r)
    emit("s_waitcnt vmcnt(24) lgkmcnt(0)")
    emit("s_barrier")
    if "copypar" in OPTS:  # (with nolds) both register sets hold block 0: every stage multiplies real data
        saved = set(OPTS)
        OPTS.discard("nolds"), OPTS.discard("nolds_a"), OPTS.discard("nolds_b")
        out.extend(all_reads(0, 0))
        OPTS.update(saved)
        emit("s_waitcnt lgkmcnt(0)")
        for k in range(32):
            emit("v_mov_b32 v%d, v%d" % (AF[1] + k, AF[0] + k))
            emit("v_mov_b32 v%d, v%d" % (BF[1] + k, BF[0] + k))
    else:
        out.extend(all_reads(0, 0))
    if es == 1:
        emit("s_waitcnt lgkmcnt(0)")
        out.extend(xor_tiles(0))
    emit("s_cmp_eq_u32 s46, 0")
    emit("s_cbranch_scc1 .LW4_TAIL_%=")
    emit(".LW4_LOOP_%=:")
    for st in range(4):
        stage(st, True, True, 2, loop_tail=".LW4_LOOP_%=" if st == 3 else None)
    emit(".LW4_TAIL_%=:")
    for st in range(4):
        stage(st, False, st < 3, max(2 - st, 0))
    # the results of the last MFMAs must have been written before anything reads the accumulators, and every wave
    # must have taken its last fragments before the ring is overwritten with them
    emit("s_nop 15")
    emit("s_nop 15")
    emit("s_waitcnt vmcnt(0) lgkmcnt(0)")
    emit("s_barrier")
    out.extend(dump(0))
    emit("s_mov_b32 m0, s49")
    return out




def dump(half):
    """Accumulators of column tiles 4*half .. 4*half+3 to the wave's LDS region as a 128 x 64 row-major block: tile
    (jt, it) holds rows 16*it.. and columns 16*(jt%4)..; v26 = the lane's address for tile (0, 0)."""
    out = []
    for jt in range(4 * half, 4 * half + 4):
        for it in range(8):
            acc = (jt * 8 + it) * 4
            out.append("ds_write_b128 v26, a[%d:%d] offset:%d" % (acc, acc + 3, it * 16 * DUMP_PITCH + (jt % 4) * 64))
    out.append("s_waitcnt lgkmcnt(0)")
    return out


def main():
    path = sys.argv[1]
    with open(path, "w") as f:
        f.write("// generated by gen_gemm_w4_mainloop.py -- do not edit\n")
        if OPTS:  # a measurement build: the library's sources refuse this text
            f.write('#define GCMI_W4_EXPERIMENT_OPTS "%s"\n' % ",".join(sorted(OPTS)))
        for name, es, tb in (("BF16", 2, False), ("BF16_TB", 2, True), ("I8", 1, False)):
            lines = gen(es, tb)
            f.write("#define GCMI_W4_ASM_%s \\\n" % name)
            f.write(" \\\n".join('  "%s\\n"' % ln for ln in lines))
            f.write("\n\n")
        f.write("#define GCMI_W4_ASM_DUMP_HI \\\n")
        f.write(" \\\n".join('  "%s\\n"' % ln for ln in dump(1)))
        f.write("\n\n")
        regs = ['"v%d"' % r for r in range(32, 160)] + ['"a%d"' % r for r in range(256)]
        f.write("#define GCMI_W4_CLOBBERS %s\n" % ", ".join(regs))


if __name__ == "__main__":
    main()
