#!/usr/bin/env python3
"""Writes gemm_wide_steps.inc: the K loop of the 256x384x32 GEMM tile as inline assembly.

Why assembly: a wavefront of this tile holds 128x96 of the output, 192 accumulator registers of the 256 it may
have, and the compiler, asked to keep them next to the kernel's other state, parks accumulators in scratch inside
the main loop.  Here the accumulators are operands tied to the C++ variables, the fragments live in registers
named outright (v224..v252, declared clobbered), and every instruction of the loop is placed by hand.  The whole
K loop of a tile is ONE asm statement per group of wavefronts, loop counter and K offsets in scalar registers:
code the compiler places between two statements may use the fragment registers (they are only clobbers to it),
and a value it reloads into one of them from scratch arrives behind the direct loads in flight, on top of a
fragment.

What bounds these GEMMs is the CU's vector memory path, which holds a limited number of requests to L2 at a time
whatever their size: the operands are therefore fetched in whole 128-byte lines.  B's rows (768 bytes per tile) are
lines anyway; A is loaded 64 columns of K at a time, so that a row's piece is one line, into a ring of its own.

Tile geometry (must match the set-up in gemm_kernel_dma.h):
  LDS  [A slot 0..1: 256 rows x 128 B = 64 columns of K][B stage 0..2: 32 k rows x 768 B].
       A fragment (32 rows x 16 k): one ds_read_b128 at vA ^ (32 * k-step within the slot) + 4096 per MFMA row tile
       (16-byte pieces of a row are swizzled with bits 1..3 of the row number, which the XOR leaves alone).
       B fragment: two ds_read_b64_tr_b16 at vB[j] + 12288 per k-step of the chunk, + 3072 for the upper four k rows;
       vB[j] contains the B region's offset.
  Direct loads per wavefront: A, every second chunk, four loads of 8 rows x 128 B (voffsets a0..a3, K offset
       soffA & ~127: the slot's first column), destination m0A + slot * 32768 + q * 1024; B, every chunk, three loads
       (voffsets b0..b2, K offset chunk * dB), destination m0B + stage * 24576 + q * 1024.
  soffA = 64 bytes x the chunk whose loads go out next; it stops at the last chunk (what is loaded after that goes
  into slots nobody reads any more, from addresses inside the operands).

Order (see gemm_kernel_dma.h, "The 256x384 tile"): all eight wavefronts run the same stream.  A wavefront has
one set of fragment registers; each fragment is read again for the next k-step right behind its last use in this
one, so the reads travel under the MFMAs still to come and the second wavefront of the SIMD fills what is left.
Barrier x (passed when chunk x and, x even, A slot x/2 have landed for everyone) sits inside the second k-step of
chunk x-1, behind its first four MFMAs: the fragments read after it are the first of chunk x; behind it everyone
issues chunk x+2 of B (into the stage chunk x-1 has just left) and, x even, A slot x/2+1.
"""
import os

OPTS = set(filter(None, os.environ.get("WIDE_OPTS", "").replace("+", ",").split(",")))      # experiment switches; none set in the build

T = 224                                   # first fragment register
FA = [T + 4 * i for i in range(4)]        # A fragments, four registers each
FB = [T + 16 + 4 * j for j in range(3)]   # B fragments (lower two registers: k rows 0..3 of each half, upper two: 4..7)
TMP = T + 28
A_SLOT, B_STAGE = 256 * 128, 32 * 768
PERIOD = 12                               # chunks after which A slot (c/2 % 2), B stage (c % 3) and parity repeat


def v(first, count):
    return "v[%d:%d]" % (first, first + count - 1)


def reads(c, kk):
    """Load phase: all fragments of k-step kk of chunk c.  Order: B0, A0..A3, B1, B2."""
    slot, stage, kp = (c // 2) % 2, c % 3, 2 * (c % 2) + kk
    out = []
    a_addr = "%[vA]"
    if kp:
        out.append("v_xor_b32 v%d, %d, %%[vA]" % (TMP, 32 * kp))
        a_addr = "v%d" % TMP
    def b(j):
        off = stage * B_STAGE + kk * 16 * 768
        return ["ds_read_b64_tr_b16 %s, %%[vB%d] offset:%d" % (v(FB[j], 2), j, off),
                "ds_read_b64_tr_b16 %s, %%[vB%d] offset:%d" % (v(FB[j] + 2, 2), j, off + 4 * 768)]
    out += b(0)
    for i in range(4):
        out.append("ds_read_b128 %s, %s offset:%d" % (v(FA[i], 4), a_addr, slot * A_SLOT + i * 4096))
    out += b(1) + b(2)
    if "noread" in OPTS:       # timing experiment: no fragment reads (wrong results)
        return []
    return out


# position of each fragment's last read in the order above, for the waits: B0 lo/hi 0,1; A0..A3 2..5; B1 6,7; B2 8,9
LAST_A = [2, 3, 4, 5]
LAST_B = [1, 7, 9]


def batch(x):
    """The direct loads issued behind barrier x: chunk x+2 of B, and with x even A slot x/2+1.  Each entry is the
    instructions of one load."""
    out = []
    if "noload" in OPTS:       # timing experiment: no direct loads in the loop (wrong results)
        return [["s_nop 0"]]
    if x % 2 == 0:
        slot = (x // 2 + 1) % 2
        for q in range(4):
            pre = ["s_and_b32 vcc_lo, %[soffA], 0xffffff80"] if q == 0 else []
            out.append(pre + ["s_add_u32 m0, %%[m0A], %d" % (slot * A_SLOT + q * 1024),
                              "buffer_load_dwordx4 %%[a%d], %%[rA], vcc_lo offen lds" % q])
    stage = (x + 2) % 3
    for q in range(3):
        pre = ["s_lshr_b32 vcc_hi, %[soffA], 6", "s_mul_i32 vcc_hi, vcc_hi, %[dB]"] if q == 0 else []
        out.append(pre + ["s_add_u32 m0, %%[m0B], %d" % (stage * B_STAGE + q * 1024),
                          "buffer_load_dwordx4 %%[b%d], %%[rB], vcc_hi offen lds" % q])
    return out


class Wave:
    """Instruction stream of one wavefront with the bookkeeping of its outstanding LDS reads: a read of fragment f is
    appended with read(); need(f) emits the s_waitcnt that makes sure f has arrived (reads return in order)."""

    def __init__(self):
        self.out = []
        self.pending = []          # fragment names of the reads still possibly outstanding, oldest first

    def emit(self, *ins):
        self.out += ins

    def read(self, frag, ins):
        self.out.append(ins)
        self.pending.append(frag)

    def need(self, frag):
        if frag in self.pending:
            last = len(self.pending) - 1 - self.pending[::-1].index(frag)
            younger = len(self.pending) - 1 - last
            self.out.append("s_waitcnt lgkmcnt(%d)" % younger)
            self.pending = self.pending[last + 1:]

    def drain(self):
        if self.pending:
            self.out.append("s_waitcnt lgkmcnt(0)")
            self.pending = []


def frag_reads(c, kk):
    """The reads of k-step kk of chunk c, by fragment: {"A0".."A3": [ins], "B0".."B2": [lo, hi]} (plus the address set-up)."""
    slot, stage, kp = (c // 2) % 2, c % 3, 2 * (c % 2) + kk
    setup = []
    a_addr = "%[vA]"
    if kp:
        setup = ["v_xor_b32 v%d, %d, %%[vA]" % (TMP, 32 * kp)]
        a_addr = "v%d" % TMP
    r = {}
    for i in range(4):
        r["A%d" % i] = ["ds_read_b128 %s, %s offset:%d" % (v(FA[i], 4), a_addr, slot * A_SLOT + i * 4096)]
    for j in range(3):
        off = stage * B_STAGE + kk * 16 * 768
        r["B%d" % j] = ["ds_read_b64_tr_b16 %s, %%[vB%d] offset:%d" % (v(FB[j], 2), j, off),
                        "ds_read_b64_tr_b16 %s, %%[vB%d] offset:%d" % (v(FB[j] + 2, 2), j, off + 4 * 768)]
    return setup, r


def issue(w, frag, reads):
    if "noread" in OPTS:       # timing experiment: no fragment reads (wrong results)
        return
    for ins in reads[frag]:
        w.read(frag, ins)


def mfma(w, i, j):
    w.need("A%d" % i)
    w.need("B%d" % j)
    if "nomfma" not in OPTS:      # (timing experiment: no arithmetic)
        w.emit("v_mfma_f32_32x32x16_f16 %%[c%d%d], %s, %s, %%[c%d%d]" % (i, j, v(FB[j], 4), v(FA[i], 4), i, j))


def landed(x):
    """Own loads that must have landed before barrier x: everything but the batch issued behind barrier x-1."""
    return "s_waitcnt vmcnt(%d)" % (3 if x % 2 == 0 else 7)


# Behind the loads of barrier x (chunk x+2): on to chunk x+3 if there is one; `left` counts the chunks not yet
# finished, the one the barrier sits in included: x = nk - left + 1.
ADVANCE = ["s_cmp_gt_u32 %[left], 4",
           "s_cselect_b32 vcc_lo, 64, 0",
           "s_add_u32 %[soffA], %[soffA], vcc_lo"]


def kstep(w, c, kk, barrier):
    """The twelve MFMAs of k-step kk of chunk c, B fragment by B fragment.  Every fragment is read again, for the
    k-step that follows, right behind its last use, so that the reads travel under the MFMAs still to come:
    B0 behind the first four, B1 behind the next four, A0..A3 one by one in the last four, B2 at the end.
    With `barrier` (second k-step of a chunk) the next k-step's fragments lie in the next chunk's stage: barrier c+1
    sits behind the first four MFMAs, and the direct loads it releases go out between the MFMAs after it."""
    nc, nkk = (c, 1) if kk == 0 else (c + 1, 0)
    setup, nxt = frag_reads(nc % PERIOD, nkk)
    loads = batch((c + 1) % PERIOD) if barrier else []
    after = {4 + (k * 8) // len(loads): k for k in range(len(loads))} if loads else {}
    n = 0
    for j in range(3):
        for i in range(4):
            mfma(w, i, j)
            if n in after:
                w.emit(*loads[after[n]])
            if j == 2:
                issue(w, "A%d" % i, nxt)
            n += 1
        if j == 0:
            if barrier:
                w.drain()                       # own reads of this chunk's stage are done: it is refilled behind the barrier
                w.emit(landed(c + 1), "s_barrier")
            w.emit(*setup)
            issue(w, "B0", nxt)
        elif j == 1:
            issue(w, "B1", nxt)
        else:
            issue(w, "B2", nxt)


def loop():
    """The whole K loop of a tile, the same for every wavefront: barrier 0, its loads, the first fragments; then chunk
    after chunk, twelve to a round of the loop."""
    w = Wave()
    w.emit(landed(0), "s_barrier")
    w.emit(*[ins for load in batch(0) for ins in load])
    w.emit("s_cmp_gt_u32 %[left], 3", "s_cselect_b32 vcc_lo, 64, 0", "s_add_u32 %[soffA], %[soffA], vcc_lo")
    setup, first = frag_reads(0, 0)
    w.emit(*setup)
    for f in ("B0", "B1", "A0", "A1", "A2", "A3", "B2"):       # the order in which the loop leaves them outstanding
        issue(w, f, first)
    w.emit("LOOP_%=:")
    entry = list(w.pending)
    for c in range(PERIOD):
        kstep(w, c, 0, False)
        kstep(w, c, 1, True)
        w.emit(*ADVANCE)
        w.emit("s_sub_u32 %[left], %[left], 1", "s_cmp_eq_u32 %[left], 0")
        w.emit("s_cbranch_scc1 DONE_%=" if c < PERIOD - 1 else "s_cbranch_scc0 LOOP_%=")
    assert w.pending == entry, (w.pending, entry)       # the loop's entry state repeats
    w.emit("DONE_%=:", "s_waitcnt lgkmcnt(0)")          # (fragments of a chunk past the end: read, never used)
    return w.out + TAIL


TAIL = ["s_nop 7", "s_nop 4"]        # the last MFMAs' results are not the compiler's to touch before they are written

# ---------------------------------------------------------------------------------------------------------------
# The 256x192 tile in whole cache lines (DmaCfg<256, 192, 64, 4, 2, ...>): eight wavefronts of 64x96 (96 accumulator
# registers), so there is room for two sets of fragments: the reads of a k-step's fragments go out between the MFMAs
# of the k-step before.  LDS: [A slot 0..2: 256 rows x 128 B = 64 columns of K][B stage 0..3: 32 k rows x 384 B].
# A chunk is 32 columns of K (two k-steps); barrier x, passed when chunk x of B and, x even, A slot x/2 have landed
# for everyone, sits in front of the second k-step of chunk x-1, whose reads are the first of chunk x; behind it
# everyone issues chunk x+3 of B (two loads: 1 KiB and, lower half of the wavefront only, 512 bytes) and, x even,
# A slot x/2+2 (four loads).  Loads therefore have three chunks (B) and four (A) to land in, more than the latency
# of a miss; with two A slots they had two, and every slot waited for its slowest line.
F2 = 200                                       # fragment sets: set s at F2 + 20 s: A0, A1 (four registers each), B0..B2
TMP2 = 240
A_SLOT2, B_STAGE2, B_BASE2 = 256 * 128, 32 * 384, 3 * 256 * 128
PERIOD2 = 12


def fa2(s, i):
    return F2 + 20 * s + 4 * i


def fb2(s, j):
    return F2 + 20 * s + 8 + 4 * j


def frag_reads2(c, kk, s):
    """Reads of k-step kk of chunk c into fragment set s: one group of instructions per fragment (A0, A1, B0, B1, B2)."""
    aslot, bstage, kp = (c // 2) % 3, c % 4, 2 * (c % 2) + kk
    groups = []
    pre = []
    a_addr, a_off = "%[vA]", aslot * A_SLOT2
    if a_off + 4096 > 65535:                     # beyond the instruction's 16-bit offset: through a register
        pre.append("v_add_u32 v%d, %d, %%[vA]" % (TMP2, a_off))
        a_addr, a_off = "v%d" % TMP2, 0
    if kp:
        pre.append("v_xor_b32 v%d, %d, %s" % (TMP2, 32 * kp, a_addr))
        a_addr = "v%d" % TMP2
    for i in range(2):
        groups.append((pre if i == 0 else []) + ["ds_read_b128 %s, %s offset:%d" % (v(fa2(s, i), 4), a_addr, a_off + i * 4096)])
    for j in range(3):
        off = bstage * B_STAGE2 + kk * 16 * 384
        groups.append(["ds_read_b64_tr_b16 %s, %%[vB%d] offset:%d" % (v(fb2(s, j), 2), j, off),
                       "ds_read_b64_tr_b16 %s, %%[vB%d] offset:%d" % (v(fb2(s, j) + 2, 2), j, off + 4 * 384)])
    return groups


def batch2(x):
    """Direct loads behind barrier x: chunk x+3 of B and, x even, A slot x/2+2.  soffA is 64 bytes x the B chunk."""
    out = []
    if "noload" in OPTS:
        return [["s_nop 0"]]
    if x % 2 == 0:
        slot = (x // 2 + 2) % 3
        for q in range(4):
            pre = ["s_add_u32 vcc_lo, %[soffA], 64", "s_and_b32 vcc_lo, vcc_lo, 0xffffff80", "s_min_u32 vcc_lo, vcc_lo, %[last]"] if q == 0 else []
            out.append(pre + ["s_add_u32 m0, %%[m0A], %d" % (slot * A_SLOT2 + q * 1024),
                              "buffer_load_dwordx4 %%[a%d], %%[rA], vcc_lo offen lds" % q])
    stage = (x + 3) % 4
    out.append(["s_lshr_b32 vcc_hi, %[soffA], 6", "s_mul_i32 vcc_hi, vcc_hi, %[dB]",
                "s_add_u32 m0, %%[m0B], %d" % (stage * B_STAGE2),
                "buffer_load_dwordx4 %[b0], %[rB], vcc_hi offen lds"])
    out.append(["s_add_u32 m0, %%[m0B], %d" % (stage * B_STAGE2 + 1024),
                "s_mov_b64 exec, 0xffffffff",
                "buffer_load_dwordx4 %[b1], %[rB], vcc_hi offen lds",
                "s_mov_b64 exec, -1"])
    return out


def kstep2(w, c, kk):
    """Six MFMAs of k-step kk of chunk c on fragment set kk; the reads of the next k-step go out between them, and
    in front of a chunk's second k-step sits barrier c+1 with its loads behind."""
    s = kk
    nc, nkk = (c, 1) if kk == 0 else (c + 1, 0)
    reads = [] if "noread" in OPTS else frag_reads2(nc % PERIOD2, nkk, 1 - s)
    names = ["A0", "A1", "B0", "B1", "B2"]
    now = []
    if kk == 1:
        w.drain()                                            # chunk c's last reads (this k-step's fragments) are done
        w.emit("s_waitcnt vmcnt(8)", "s_barrier")            # chunk c+1 has landed for everyone
        now = batch2((c + 1) % PERIOD2)
    n = 0
    for j in range(3):
        for i in range(2):
            w.need("%s.A%d" % (s, i))
            w.need("%s.B%d" % (s, j))
            if "nomfma" not in OPTS:
                w.emit("v_mfma_f32_32x32x16_f16 %%[c%d%d], %s, %s, %%[c%d%d]" % (i, j, v(fb2(s, j), 4), v(fa2(s, i), 4), i, j))
            if n < len(reads):
                for ins in reads[n]:
                    if ins.startswith("ds_read"):
                        w.read("%s.%s" % (1 - s, names[n]), ins)
                    else:
                        w.emit(ins)
            if n < len(now):
                w.emit(*now[n])
            n += 1


def loop192():
    w = Wave()
    w.emit("s_waitcnt vmcnt(8)", "s_barrier")                # barrier 0: chunk 0 of B, A slot 0
    for load in batch2(0):
        w.emit(*load)
    w.emit("s_cmp_gt_u32 %[left], 4", "s_cselect_b32 vcc_lo, 64, 0", "s_add_u32 %[soffA], %[soffA], vcc_lo")
    if "noread" not in OPTS:
        for name, g in zip(["A0", "A1", "B0", "B1", "B2"], frag_reads2(0, 0, 0)):
            for ins in g:
                w.read("0." + name, ins)
    w.emit("LOOP_%=:")
    entry = list(w.pending)
    for c in range(PERIOD2):
        kstep2(w, c, 0)
        kstep2(w, c, 1)
        # behind the loads of barrier c+1 (chunk c+4 of B): on while there is another chunk
        w.emit("s_cmp_gt_u32 %[left], 5", "s_cselect_b32 vcc_lo, 64, 0", "s_add_u32 %[soffA], %[soffA], vcc_lo")
        w.emit("s_sub_u32 %[left], %[left], 1", "s_cmp_eq_u32 %[left], 0",
               "s_cbranch_scc1 DONE_%=" if c < PERIOD2 - 1 else "s_cbranch_scc0 LOOP_%=")
    assert w.pending == entry, (w.pending, entry)
    w.emit("DONE_%=:", "s_waitcnt lgkmcnt(0)")
    return w.out + TAIL


STATE_OPS = '[soffA] "+s"(soffA), [left] "+s"(left)'
CLOBBERS2 = ", ".join('"v%d"' % r for r in range(F2, TMP2 + 1)) + ', "vcc", "scc", "memory"'
ACC_OPS2 = ", ".join('[c%d%d] "+v"(acc[%d][%d])' % (i, j, i, j) for i in range(2) for j in range(3))
IN_OPS2 = ('[vA] "v"(w.vA), [vB0] "v"(w.vB[0]), [vB1] "v"(w.vB[1]), [vB2] "v"(w.vB[2]), '
           '[a0] "v"(w.a[0]), [a1] "v"(w.a[1]), [a2] "v"(w.a[2]), [a3] "v"(w.a[3]), [b0] "v"(w.b[0]), [b1] "v"(w.b[1]), '
           '[rA] "s"(w.rA), [rB] "s"(w.rB), [m0A] "s"(w.m0A), [m0B] "s"(w.m0B), [dB] "s"(w.dB), [last] "s"(last)')


def function192(name, body):
    text = "\\n\\t".join(body)
    lines = ["// soffA: 64 bytes x the chunk (32 columns of K) of B whose loads go out next (A slots 0 and 1 and chunks 0 to 2 of B are the",
             "// caller's); the A slot that goes out with every second one begins one chunk later, held at `last`, the byte offset of the",
             "// last slot there is; left: chunks to compute.",
             "__device__ __forceinline__ void %s(floatx16 (&acc)[2][3], const WideOperands& w, uint32_t soffA, uint32_t left, uint32_t last) {" % name,
             '  asm volatile("%s"' % text,
             "               : %s, %s" % (ACC_OPS2, STATE_OPS),
             "               : %s" % IN_OPS2,
             "               : %s);" % CLOBBERS2,
             "}"]
    return "\n".join(lines)


CLOBBERS = ", ".join('"v%d"' % r for r in range(T, TMP + 1)) + ', "vcc", "scc", "memory"'
ACC_OPS = ", ".join('[c%d%d] "+v"(acc[%d][%d])' % (i, j, i, j) for i in range(4) for j in range(3))
IN_OPS = ('[vA] "v"(w.vA), [vB0] "v"(w.vB[0]), [vB1] "v"(w.vB[1]), [vB2] "v"(w.vB[2]), '
          '[a0] "v"(w.a[0]), [a1] "v"(w.a[1]), [a2] "v"(w.a[2]), [a3] "v"(w.a[3]), [b0] "v"(w.b[0]), [b1] "v"(w.b[1]), [b2] "v"(w.b[2]), '
          '[rA] "s"(w.rA), [rB] "s"(w.rB), [m0A] "s"(w.m0A), [m0B] "s"(w.m0B), [dB] "s"(w.dB)')


def function(name, body):
    text = "\\n\\t".join(body)
    lines = ["// soffA: 64 bytes x the chunk whose loads go out next (chunks 0 and 1 and A slot 0 are the caller's); left: chunks to compute.",
             "__device__ __forceinline__ void %s(floatx16 (&acc)[4][3], const WideOperands& w, uint32_t soffA, uint32_t left) {" % name,
             '  asm volatile("%s"' % text,
             "               : %s, %s" % (ACC_OPS, STATE_OPS),
             "               : %s" % IN_OPS,
             "               : %s);" % CLOBBERS,
             "}"]
    return "\n".join(lines)


def main():
    out = ["// Generated by gen_wide_steps.py; do not edit.  The K loop of the 256x384x32 tile (see that script).",
           "#pragma once", "", function("wideLoop", loop()), "", function192("pairLoop192", loop192()), ""]
    path = os.environ.get("WIDE_OUT") or os.path.join(os.path.dirname(os.path.abspath(__file__)), "gemm_wide_steps.inc")
    with open(path, "w") as f:
        f.write("\n".join(out))


if __name__ == "__main__":
    main()
