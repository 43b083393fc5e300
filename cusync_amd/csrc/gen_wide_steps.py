#!/usr/bin/env python3
"""Writes gemm_wide_steps.inc: the K-chunk steps of the 256x384x32 GEMM tile as inline assembly.

Why assembly: a wavefront of this tile holds 128x96 of the output, 192 accumulator registers of the 256 it may
have, and the compiler, asked to keep them next to the kernel's other state, parks accumulators in scratch inside
the main loop.  Here the accumulators are operands tied to the C++ variables, the fragments live in registers
named outright (v224..v252, declared clobbered), and every instruction of a chunk is placed by hand.

Tile geometry (must match DmaCfg<256, 384, 32, 2, 4, 3, 2, false, false, true>):
  LDS  [A stage 0..2: 256 rows x 64 B][B stage 0..2: 32 rows x 768 B]; an A fragment is one ds_read_b128 at
  vA (+ 2048 per 32-row MFMA tile; k-step 1 at vA ^ 32), a B fragment two ds_read_b64_tr_b16 at vB[j]
  (+ 12288 per k-step, + 3072 for the upper four k rows); vB[j] already contains the B region's offset.
  Direct loads per wavefront and chunk: two of A (rows 16 apart) and three of B, destination M0 =
  m0A + stage * 16384 + q * 1024 and m0B + stage * 24576 + q * 1024; the chunk's K offset comes in through the
  scalar offsets (soffA bytes along a row of A, soffB bytes down the rows of B).

The wavefronts are two groups, one phase apart (see gemm_kernel_dma.h, "Alternating order"):
  group A, chunk c:  wait own loads of c | barrier c | read k0 | mfma k0 + loads of c+2 | read k1 | mfma k1
  group B, chunk c:  read k0 | mfma k0 | read k1 | wait LDS, own loads of c+1 | barrier c+1 | mfma k1 + loads of c+3
The whole K loop of a tile is ONE asm statement per group, loop counter and K offsets in scalar registers: code
the compiler places between two statements may use the fragment registers (they are only clobbers to it), and
a value it reloads into one of them from scratch arrives behind the direct loads in flight, on top of a fragment.
"""
import os

T = 224                                   # first fragment register
FA = [T + 4 * i for i in range(4)]        # A fragments, four registers each
FB = [T + 16 + 4 * j for j in range(3)]   # B fragments (lower two registers: k rows 0..3, upper two: 4..7 of each half)
TMP = T + 28
A_STAGE, B_STAGE = 256 * 64, 32 * 768
LOADS_AFTER = {0: ("A", 0), 2: ("A", 1), 4: ("B", 0), 7: ("B", 1), 9: ("B", 2)}   # direct load issued behind MFMA number ...


def v(first, count):
    return "v[%d:%d]" % (first, first + count - 1)


def reads(stage, kk):
    """Load phase: all fragments of k-step kk.  Order: B0, A0..A3, B1, B2."""
    out = []
    a_addr = "%[vA]" if kk == 0 else "v%d" % TMP
    if kk == 1:
        out.append("v_xor_b32 v%d, 32, %%[vA]" % TMP)
    def b(j):
        off = stage * B_STAGE + kk * 16 * 768
        return ["ds_read_b64_tr_b16 %s, %%[vB%d] offset:%d" % (v(FB[j], 2), j, off),
                "ds_read_b64_tr_b16 %s, %%[vB%d] offset:%d" % (v(FB[j] + 2, 2), j, off + 4 * 768)]
    out += b(0)
    for i in range(4):
        out.append("ds_read_b128 %s, %s offset:%d" % (v(FA[i], 4), a_addr, stage * A_STAGE + i * 2048))
    out += b(1) + b(2)
    return out


# position of each fragment's last read in the order above, for the waits: B0 lo/hi 0,1; A0..A3 2..5; B1 6,7; B2 8,9
LAST_A = [2, 3, 4, 5]
LAST_B = [1, 7, 9]


def mfmas(load_stage=None, waits=True):
    """Compute phase: 12 MFMAs, B fragment by B fragment; with load_stage the chunk's five direct loads between them."""
    out = ["s_setprio 1"]
    allowed = 10          # reads that may still be outstanding
    n = 0
    for j in range(3):
        for i in range(4):
            if waits:
                need = 9 - max(LAST_A[i], LAST_B[j])
                if need < allowed:
                    out.append("s_waitcnt lgkmcnt(%d)" % need)
                    allowed = need
            out.append("v_mfma_f32_32x32x16_f16 %%[c%d%d], %s, %s, %%[c%d%d]" % (i, j, v(FB[j], 4), v(FA[i], 4), i, j))
            if load_stage is not None and n in LOADS_AFTER:
                which, q = LOADS_AFTER[n]
                if which == "A":
                    out.append("s_add_u32 m0, %%[m0A], %d" % (load_stage * A_STAGE + q * 1024))
                    out.append("buffer_load_dwordx4 %%[a%d], %%[rA], %%[soffA] offen lds" % q)
                else:
                    out.append("s_add_u32 m0, %%[m0B], %d" % (load_stage * B_STAGE + q * 1024))
                    out.append("buffer_load_dwordx4 %%[b%d], %%[rB], %%[soffB] offen lds" % q)
            n += 1
    out.append("s_setprio 0")
    return out


TAIL = ["s_nop 7", "s_nop 4"]        # the last MFMAs' results are not the compiler's to touch before they are written


def step_a(stage):
    body = ["s_waitcnt vmcnt(5)", "s_barrier"]
    body += reads(stage, 0) + mfmas(load_stage=(stage + 2) % 3) + reads(stage, 1) + mfmas() + TAIL
    return body


def step_b(stage):
    body = reads(stage, 0) + mfmas() + reads(stage, 1)
    body += ["s_waitcnt lgkmcnt(0)", "s_waitcnt vmcnt(5)", "s_barrier"]
    body += mfmas(load_stage=stage, waits=False) + TAIL
    return body


def loads(load_stage):
    out = []
    for which, q in (("A", 0), ("A", 1), ("B", 0), ("B", 1), ("B", 2)):
        if which == "A":
            out += ["s_add_u32 m0, %%[m0A], %d" % (load_stage * A_STAGE + q * 1024), "buffer_load_dwordx4 %%[a%d], %%[rA], %%[soffA] offen lds" % q]
        else:
            out += ["s_add_u32 m0, %%[m0B], %d" % (load_stage * B_STAGE + q * 1024), "buffer_load_dwordx4 %%[b%d], %%[rB], %%[soffB] offen lds" % q]
    return out


# After the loads of a step: the K offsets move on to the next chunk while there is one (afterwards the last chunk is
# loaded again, into a stage nobody reads any more, so that no address ever leaves the operands).
ADVANCE = ["s_cmp_lg_u32 %[adv], 0",
           "s_cselect_b32 vcc_lo, 64, 0",
           "s_cselect_b32 vcc_hi, %[dB], 0",
           "s_add_u32 %[soffA], %[soffA], vcc_lo",
           "s_add_u32 %[soffB], %[soffB], vcc_hi",
           "s_add_i32 %[adv], %[adv], -1",
           "s_max_i32 %[adv], %[adv], 0"]


def count_down(label_if_zero=None, label_if_more=None):
    out = ["s_sub_u32 %[left], %[left], 1", "s_cmp_eq_u32 %[left], 0"]
    if label_if_zero:
        out.append("s_cbranch_scc1 %s" % label_if_zero)
    if label_if_more:
        out.append("s_cbranch_scc0 %s" % label_if_more)
    return out


def loop_a():
    """The whole K loop of a tile for the first group."""
    body = ["LOOP_A_%=:"]
    for s in range(3):
        body += step_a(s)[:-len(TAIL)] + ADVANCE
        body += count_down("DONE_A_%=") if s < 2 else count_down(None, "LOOP_A_%=")
    body += ["DONE_A_%=:", "s_barrier"] + TAIL       # the second group's last barrier
    return body


def loop_b():
    """The whole K loop of a tile for the second group: barrier 0 and the loads of chunk 2 first."""
    body = ["s_waitcnt vmcnt(5)", "s_barrier"] + loads(2) + ADVANCE
    body += ["LOOP_B_%=:"]
    for s in range(3):
        body += step_b(s)[:-len(TAIL)] + ADVANCE
        body += count_down("DONE_B_%=") if s < 2 else count_down(None, "LOOP_B_%=")
    body += ["DONE_B_%=:"] + TAIL
    return body


CLOBBERS = ", ".join('"v%d"' % r for r in range(T, TMP + 1)) + ', "vcc", "scc", "memory"'
ACC_OPS = ", ".join('[c%d%d] "+v"(acc[%d][%d])' % (i, j, i, j) for i in range(4) for j in range(3))
STATE_OPS = '[soffA] "+s"(soffA), [soffB] "+s"(soffB), [left] "+s"(left), [adv] "+s"(adv)'
IN_OPS = ('[vA] "v"(w.vA), [vB0] "v"(w.vB[0]), [vB1] "v"(w.vB[1]), [vB2] "v"(w.vB[2]), '
          '[a0] "v"(w.a[0]), [a1] "v"(w.a[1]), [b0] "v"(w.b[0]), [b1] "v"(w.b[1]), [b2] "v"(w.b[2]), '
          '[rA] "s"(w.rA), [rB] "s"(w.rB), [m0A] "s"(w.m0A), [m0B] "s"(w.m0B), [dB] "s"(w.dB)')


def function(name, body):
    text = "\\n\\t".join(body)
    lines = ["// soffA, soffB: K offsets (bytes along a row of A, bytes down the rows of B) of the chunk to load next; left: chunks to",
             "// compute; adv: how many more times the offsets move on by one chunk.",
             "__device__ __forceinline__ void %s(floatx16 (&acc)[4][3], const WideOperands& w, uint32_t soffA, uint32_t soffB, uint32_t left, uint32_t adv) {" % name]
    lines.append('  asm volatile("%s"' % text)
    lines.append("               : %s, %s" % (ACC_OPS, STATE_OPS))
    lines.append("               : %s" % IN_OPS)
    lines.append("               : %s);" % CLOBBERS)
    lines.append("}")
    return "\n".join(lines)


def main():
    out = ["// Generated by gen_wide_steps.py; do not edit.  The K loop of the 256x384x32 tile (see that script).",
           "#pragma once", "",
           function("wideLoopA", loop_a()), "", function("wideLoopB", loop_b()), ""]
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gemm_wide_steps.inc")
    with open(path, "w") as f:
        f.write("\n".join(out))


if __name__ == "__main__":
    main()
