#!/usr/bin/env python3
"""Generates gmm_tile_asm.inc: the per-tile main loop and epilogue of the MFMA
grouped GEMM kernels as hand-scheduled gfx950 assembly.

    python gen_tile_asm.py > gmm_tile_asm.inc      (build.py does this)

Why generated assembly: the loop keeps 256 accumulator registers, two sets of
MFMA operand fragments and sixteen in-flight direct-to-LDS copies alive at once.
Written as C++ the compiler spills inside the loop, and every spill reload waits
on the vector-memory counter that the asynchronous copies also use, which stalls
the pipeline.  Here every register is named, so nothing is spilled and the issue
order is exactly the one below.

One block computes one 256 x 256 output tile with 4 waves (2 x 2, 128 x 128 per
wave, 8 x 8 MFMA blocks of 16 x 16); variants for 128 x 256 and 64 x 256 tiles
(group remainders, small groups) and for fp16 instead of bf16 elements.  The MFMA
is v_mfma_f32_16x16x32: per FLOP it moves half the accumulator data of the
32 x 32 x 16 shape through the register file, and in a register-only loop on
operands drawn like the benchmark's it sustains 1960-2050 TFLOP/s where
32 x 32 x 16 sustains 1790-1810 (the clock follows the power drawn):

  * K is walked in tiles of 64; A and B tiles are copied global -> LDS by
    buffer_load_dwordx4 ... lds (no registers involved) into two buffers (three
    for the 128- and 64-row tiles, which have the LDS room and need the deeper
    prefetch);
  * an operand that is contiguous along K lives in LDS as [row][64 k] with its
    16-byte chunks XOR-swizzled (conflict-free ds_read_b128 fragments); one that
    is contiguous along M / N lives as [k][256] in blocks of two k rows with a
    32-byte pad, read with ds_read_b64_tr_b16 (the LDS transposes 4 x 16 blocks);
  * a K tile is four steps: (k 0..31, upper half of the wave's rows), (k 0..31,
    lower half), (k 32..63, upper), (k 32..63, lower).  A step issues 8 tm
    v_mfma_f32_16x16x32 (tm = 4 for the 256-row tile) and, between them, the
    fragment reads the following steps need -- the A fragments of the next step
    into the other of two A register sets, the B fragments of the next k half
    into the other of two B sets -- and its share of the copies of the next
    tiles.  LDS reads complete in order: every MFMA waits (lgkmcnt) only until
    its own operands have arrived;
  * the loop body exists twice: K tiles whose copies are neither the last tile of
    the range nor past it use the copy offsets as they are; the others select
    per copy between the normal offsets, the last tile's offsets and "out of
    range" (a buffer load that fetches nothing and writes zeros);
  * one s_barrier per K tile, placed after step 2 so that step 3's MFMAs run
    while the barrier's stragglers arrive and the first fragments of the next
    tile (its B fragments of k 0..31 and the A fragments of its step 0) are
    fetched under them;
  * epilogue: the MFMA operands are swapped so a lane owns 4 consecutive columns;
    it packs them (v_cvt_pk_bf16_f32; fp32 goes as it is), stages the wave's block
    in LDS and writes 16 bytes per lane: 256 contiguous bytes per row (512 for
    fp32); a chunk that a group boundary cuts (jagged columns) goes out element
    by element.

Registers:
  a[0:255]     accumulators, 16 x 16 block (i, j) at a[(8 i + j) 4 ...]
  v[0:15]      A fragments set 0 (four of 16 rows x 32 k), v[16:31] set 1,
  v[32:63]     B fragments set 0 (eight of 16 columns x 32 k), v[64:95] set 1
  v[96:119]    temporaries, per-buffer fragment addresses of the 3-buffer variants
  inputs are pinned by the C++ wrapper to v[120:191] and s[28:55] (see GmmTileRegs).
"""
import sys

# copies (of the 16 per K tile and wave) issued in: step 3 right after the barrier, then steps 0, 1, 2
# of the next K tile; the tile must have landed at that tile's barrier (end of its step 2).
COPY_SCHEDULE = (8, 8, 0, 0)
# Order of the copies of a K tile: B first.  B is the operand that streams from HBM (every group has its
# own), A is re-read by every tile column and mostly comes out of the Infinity Cache: the copies issued
# first have the most time to land.
B_COPIES_FIRST = 1
# L2 prefetch: in every K tile each wave issues one plain dword load per operand whose lanes touch the cache
# lines of K tile kt + TOUCH_DIST (the result is discarded).  A direct-to-LDS copy can only be issued one K
# tile ahead (two LDS buffers), which is less than the latency of HBM; the touches bring the lines into the
# L2 ahead of time so that the copies hit.  0 = off.  TOUCH_OPS: which operands ("a", "b").
TOUCH_DIST = 3
TOUCH_OPS = "b"

PITCH = 272           # bytes per staged row of 128 bf16 (256 + 16: shifts banks per row)
PITCH32 = 528         # ... of 128 fp32 (512 + 16)
PITCH_ACT = 144       # ... of the 64 gated values a wave's 128 columns give (128 + 16)
TR_BLOCK = 1056       # two k rows of 512 bytes + 32 bytes pad: the four blocks that 16 lanes of a transposing read
                      # address lie 8 banks apart (32 consecutive banks), the next 16 lanes' blocks on the other 32
KC_STAGE = 256 * 64 * 2
TR_STAGE = 32 * TR_BLOCK
STAGE_BYTES = 4 * 128 * PITCH

# ---- fixed register map: one wave per SIMD (128 x 128 per wave, 256 accumulators), the wave owns all 512
# registers of a lane.
STAGES_SHORT = 3         # LDS buffers of the 128- and 64-row tiles
V_AF = [0, 16]           # A fragment sets (up to 4 fragments x 4 registers each)
V_BF = [32, 64]          # B fragment sets (8 x 4 registers each)
V_TMP = 96               # 96..105: temporaries of the main loop (the epilogue uses the fragment registers)
V_TOUCH_DST = V_TMP + 10  # +0 / +1: where the touched dwords land (never read)
V_BUFA, V_BUFB = V_TMP + 12, V_TMP + 18  # three-buffer variants: fragment addresses per (buffer, k half), 6 + 6
V_CLOBBER = 120
V_IN = 120               # first register of the inputs the wrapper pins
V_VOA_HEAD, V_VOB_HEAD, V_VOA, V_VOB, V_VOA_TAIL, V_VOB_TAIL = (V_IN + 8 * i for i in range(6))
V_RA, V_RB = V_IN + 48, V_IN + 52   # fragment read addresses (K-contiguous operand: one per k half; else one)
V_EPI = V_IN + 56        # +0: stage write addr, +1: stage read addr, +2: store voffset, +3: row - row_lo
V_OOB = V_IN + 60        # constant 0x80000000
V_EPI2 = V_IN + 62       # +0: store voffset whatever the chunk's validity, +1: mask of valid elements if partial
V_TOUCH = V_IN + 64      # per-lane offsets of the L2 prefetch touches: +0 A, +1 B (K tile 0)
V_FIX = V_IN + 68        # A first-chunk addr, A last-chunk addr, same for B (buffer 0)
S_MASK = 28            # s[28:31] keep-mask of the first chunk of the k range, s[32:35] of the last chunk

S_RA, S_RB, S_RC = 36, 40, 44   # buffer resources
S_SC = 48                        # scalars s[48:55]
S_NK, S_ASTEP, S_BSTEP, S_LDS, S_ROWCNT, S_CSTEP, S_NVALID, S_SPARE = range(48, 56)
S_T = 56                         # temporaries s[56:79]


class Emit:
    def __init__(self):
        self.lines = []

    def __call__(self, s):
        self.lines.append(s)

    def label(self, name):
        self.lines.append(name + ":")

    def text(self):
        return "\n".join('      "%s\\n\\t"' % l for l in self.lines)


def vr(base, n=1):
    return "v%d" % base if n == 1 else "v[%d:%d]" % (base, base + n - 1)


def sr(base, n=1):
    return "s%d" % base if n == 1 else "s[%d:%d]" % (base, base + n - 1)


class Variant:
    """tm = 32-row blocks per wave: the tile is 64 tm rows (256 / 128 / 64) by 256 columns; a wave computes
    2 tm x 8 MFMA blocks of 16 x 16."""

    def __init__(self, a_tr, b_tr, out_f32, tm=4, f16=0, b_nt=0, act=0):
        """b_nt: B is copied with the non-temporal hint (a B panel that no other tile reads).
        act: SwiGLU epilogue -- of each 128 columns the first 64 are gates and the last 64 their partners;
        the tile stores silu(gate) * partner, 128 columns of a 16-bit output per 256 columns of the product."""
        self.a_tr, self.b_tr, self.out_f32, self.tm, self.f16, self.b_nt = a_tr, b_tr, out_f32, tm, f16, b_nt
        self.act = act == 1
        self.partial = act == 2      # fp32 partial tile of a tile cut along K: stored through to memory (sc1)
        assert not (self.act and (out_f32 or a_tr)) and not (self.partial and (not out_f32 or b_nt))
        self.dt = "f16" if f16 else "bf16"   # element type of A, B and of a 16-bit output
        assert tm in (1, 2, 4) and (tm == 4 or not a_tr)
        self.tn = 8                      # 16-column MFMA blocks per wave (the wave grid is 2 x 2)
        self.na = 2 * tm                 # copies of the A tile per wave and K tile
        self.nb = 8                      # ... of the B tile
        self.ncopy = self.na + self.nb
        # issue index -> copy: A copies are 0 .. na - 1, B copies na .. ncopy - 1
        self.order = list(range(self.ncopy))
        if B_COPIES_FIRST:
            self.order = list(range(self.na, self.ncopy)) + list(range(self.na))
        # 256-row tiles only: the shorter ones have a third LDS buffer (copies two K tiles ahead) and are short of
        # memory issue slots, not of prefetch distance (with touches the fine-grained workload lost 8 %)
        self.touch = [op for op in "ab" if TOUCH_DIST and op in TOUCH_OPS and tm == 4]
        self.nt = len(self.touch)
        c3 = (self.ncopy + 1) // 2
        self.sched = COPY_SCHEDULE if tm == 4 else (c3, self.ncopy - c3, 0, 0)
        # LDS buffers per operand: 2 for the 256-row tile (LDS is full), 3 for the shorter ones, whose K
        # tiles are short of MFMA work and would otherwise wait on memory latency every K tile
        self.stages = STAGES_SHORT if tm < 4 else 2
        # The loop's wait leaves (stages - 1) sets of touches in flight; the prologue issues the sets for K
        # tiles stages .. touch_dist - 1 after its copies, and the first wait of the loop must not count more
        # sets than that: touch_dist - stages + 1 >= stages - 1.
        self.touch_dist = max(TOUCH_DIST, 2 * self.stages - 2)
        self.a_stage = TR_STAGE if a_tr else (64 * tm * 128 if self.stages == 3 else KC_STAGE)
        self.b_stage = TR_STAGE if b_tr else KC_STAGE
        self.b_base = self.stages * self.a_stage   # LDS offset of B buffer 0
        self.name = "%s%s_%s_%s_m%d%s%s" % ("t" if a_tr else "k", "t" if b_tr else "k", self.dt, "f32" if out_f32 else self.dt, 64 * tm,
                                            "_bnt" if b_nt else "", "_swiglu" if act == 1 else ("_partial" if act == 2 else ""))

    def acc(self, i, j):
        """First accumulator register of the wave's 16 x 16 block (i, j), i < 2 tm, j < 8."""
        return (self.tn * i + j) * 4

    # -- one fragment (16 rows or columns x 32 k) of k half `sp` of buffer `buf` into registers d .. d + 3;
    # f = 16-row block of the wave's rows (A) / 16-column block of its columns (B)
    def frag_read(self, is_a, buf, sp, f, d):
        tr = self.a_tr if is_a else self.b_tr
        stage = self.a_stage if is_a else self.b_stage
        vaddr, vbuf = (V_RA, V_BUFA) if is_a else (V_RB, V_BUFB)
        # two buffers: the buffer is an immediate offset; three: one address register per buffer (and k
        # half), set up by the prologue, because the offsets no longer fit the 16-bit immediate
        if not tr:
            # address register per k half; 16-row blocks are 2048 bytes apart
            reg, off = (vaddr + sp, buf * stage) if self.stages == 2 else (vbuf + 2 * buf + sp, 0)
            return ["ds_read_b128 %s, %s offset:%d" % (vr(d, 4), vr(reg), off + f * 2048)]
        reg, off = (vaddr, buf * stage) if self.stages == 2 else (vbuf + 2 * buf, 0)
        o = off + sp * 16 * TR_BLOCK + f * 32
        return ["ds_read_b64_tr_b16 %s, %s offset:%d" % (vr(d, 2), vr(reg), o),
                "ds_read_b64_tr_b16 %s, %s offset:%d" % (vr(d + 2, 2), vr(reg), o + 512)]

    def a_reads(self, buf, t, order=None):
        """A fragments of step t (k half t / 2, row half t % 2) into A set t % 2: list of (tag, instructions)."""
        sp, h, st = t // 2, t % 2, t % 2
        return [(("A", st, x), self.frag_read(True, buf, sp, h * self.tm + x, V_AF[st] + 4 * x)) for x in range(self.tm)]

    def b_reads(self, buf, sp, js):
        """B fragments js of k half sp into B set sp."""
        return [(("B", sp, j), self.frag_read(False, buf, sp, j, V_BF[sp] + 4 * j)) for j in js]

    def first_reads(self, buf):
        """What step 0 of a K tile on `buf` needs, in the order its MFMAs want it: issued by the prologue and by
        step 3 of the K tile before."""
        a, b = self.a_reads(buf, 0), self.b_reads(buf, 0, range(self.tn))
        return a[:1] + b + a[1:]

    def step_reads(self, t, buf, nb):
        """Fragment reads issued during step t of a K tile on buffer `buf` (nb = buffer of the next K tile)."""
        if t == 0:
            return self.a_reads(buf, 1) + self.b_reads(buf, 1, range(0, 4))
        if t == 1:
            a = self.a_reads(buf, 2)
            return a[:1] + self.b_reads(buf, 1, range(4, 8)) + a[1:]
        if t == 2:
            return self.a_reads(buf, 3)
        return self.first_reads(nb)

    # -- MFMAs of step t: list of (operand tags, instruction)
    def mfmas(self, t):
        sp, h, st = t // 2, t % 2, t % 2
        out = []
        for x in range(self.tm):
            i = h * self.tm + x
            for j in range(self.tn):
                a = vr(V_AF[st] + 4 * x, 4)
                b = vr(V_BF[sp] + 4 * j, 4)
                c = "a[%d:%d]" % (self.acc(i, j), self.acc(i, j) + 3)
                # operands swapped: the result block is transposed, a lane owns 4 consecutive columns of a row
                out.append(((("A", st, x), ("B", sp, j)), "v_mfma_f32_16x16x32_%s %s, %s, %s, %s" % (self.dt, c, b, a, c)))
        return out

    # -- copy instruction with issue index n (0..15) of a K tile into buffer buf.
    # s_tail / s_oob: SGPR pairs (lane masks all-ones / zero): use the tail offsets / kill the copy.
    # s_ka / s_kb: SGPRs with the tile's byte offsets along K for A and B.  which: "head" or "loop".
    def dma(self, n, buf, which, s_tail, s_oob, s_ka, s_kb, tmp):
        out = []
        n = self.order[n]
        is_a = n < self.na
        i = n if is_a else n - self.na
        tr = self.a_tr if is_a else self.b_tr
        stage = self.a_stage if is_a else self.b_stage
        lbase = 0 if is_a else self.b_base
        # per wave: 8 instructions of 1 KiB each; wave w covers [w * 8 KiB, (w + 1) * 8 KiB) of the
        # stage (row-chunk layout) or blocks w * 8 .. w * 8 + 7 (transposed layout): the wave part of
        # the LDS address is in s[S_T + 20] (A) / s[S_T + 21] (B), set up by the prologue.
        lds_off = lbase + buf * stage + i * (TR_BLOCK if tr else 1024)
        s_wave = S_T + 20 + (0 if is_a else 1)
        # m0 is written first: a write of m0 needs one other instruction before the copy that uses it
        # (the selects below, an MFMA that interleave() puts in between, or a s_nop)
        out.append("s_add_u32 m0, %s, %d" % (sr(s_wave), lds_off))
        if which == "head":
            vo = (V_VOA_HEAD if is_a else V_VOB_HEAD) + i
            src = vr(vo)
        elif which == "fast":
            src = vr((V_VOA if is_a else V_VOB) + i)
        else:
            vn = (V_VOA if is_a else V_VOB) + i
            vt = (V_VOA_TAIL if is_a else V_VOB_TAIL) + i
            out.append("v_cndmask_b32_e64 %s, %s, %s, %s" % (vr(tmp), vr(vn), vr(vt), sr(s_tail, 2)))
            out.append("v_cndmask_b32_e64 %s, %s, %s, %s" % (vr(tmp), vr(tmp), vr(V_OOB), sr(s_oob, 2)))
            src = vr(tmp)
        pol = " nt" if (self.b_nt and not is_a) else ""
        out.append("buffer_load_dwordx4 %s, %s, %s offen%s lds" % (src, sr(S_RA if is_a else S_RB, 4), sr(s_ka if is_a else s_kb), pol))
        return out


def touch_group(v, op, s_mask, s_k, tmp):
    """L2 prefetch of one operand's K tile: one dword per lane, each lane on another cache line (offsets from
    the wrapper, v[V_TOUCH ..]); s_mask (SGPR pair): all-ones if that K tile exists, else nothing is fetched."""
    i = 0 if op == "a" else 1
    return ["v_cndmask_b32_e64 %s, %s, %s, %s" % (vr(tmp), vr(V_OOB), vr(V_TOUCH + i), sr(s_mask, 2)),
            "buffer_load_dword %s, %s, %s, %s offen" % (vr(V_TOUCH_DST + i), vr(tmp), sr(S_RA if op == "a" else S_RB, 4), sr(s_k))]


def m0_gaps(lines):
    """Insert the wait state between a write of m0 and a copy that follows it directly."""
    out = []
    for ins in lines:
        if ins.startswith("buffer_load") and out and out[-1].startswith("s_add_u32 m0"):
            out.append("s_nop 0")
        out.append(ins)
    return out


def fixup(e, v, which, buf):
    """Zero the k elements outside the group's range in one 16-byte chunk per row (row = thread id) of
    every operand that is contiguous along K.  which: 0 = first chunk of K tile 0, 1 = last chunk."""
    for is_a in (True, False):
        tr = v.a_tr if is_a else v.b_tr
        if tr:
            continue
        stage = v.a_stage if is_a else v.b_stage
        addr = V_FIX + (0 if is_a else 2) + which
        t = V_TMP + (0 if is_a else 4)
        ta = V_TMP + 8 + (0 if is_a else 1)
        e("v_add_u32 %s, %d, %s" % (vr(ta), buf * stage, vr(addr)))
        e("ds_read_b128 %s, %s" % (vr(t, 4), vr(ta)))
    e("s_waitcnt lgkmcnt(0)")
    for is_a in (True, False):
        tr = v.a_tr if is_a else v.b_tr
        if tr:
            continue
        stage = v.a_stage if is_a else v.b_stage
        addr = V_FIX + (0 if is_a else 2) + which
        t = V_TMP + (0 if is_a else 4)
        ta = V_TMP + 8 + (0 if is_a else 1)
        for w in range(4):
            e("v_and_b32 %s, %s, %s" % (vr(t + w), sr(S_MASK + 4 * which + w), vr(t + w)))
        e("ds_write_b128 %s, %s" % (vr(ta), vr(t, 4)))


class LdsOrder:
    """LDS reads complete in the order they were issued.  Tracks the reads that may still be in flight, so that
    an MFMA waits (s_waitcnt lgkmcnt) only until its own operands have arrived."""

    def __init__(self, pending=()):
        self.pending = list(pending)       # tags, oldest first

    def issue(self, tag, n=1):
        self.pending += [tag] * n

    def wait_for(self, tags):
        """The wait that proves every read with one of `tags` complete, or None if they already are."""
        idx = max((i for i, t in enumerate(self.pending) if t in tags), default=-1)
        if idx < 0:
            return None
        w = min(len(self.pending) - 1 - idx, 15)   # the counter has 4 bits
        self.pending = self.pending[len(self.pending) - w:] if w else []
        return w

    def clear(self):
        self.pending = []


def interleave(e, lds, mfmas, side):
    """Emit the MFMAs of a step with the side groups spread between them (after each MFMA, in order).  A
    side group is (tag, instructions): tag names the fragment a group of LDS reads fetches (None: not a
    read).  A group that starts with a write of m0 has that write moved in front of the MFMA, which then is
    the instruction the hardware wants between the write and the copy."""
    n = len(mfmas)
    slots = [[] for _ in range(n)]
    g = len(side)
    for k, grp in enumerate(side):
        slots[min(n - 1, (k * n) // max(g, 1))].append(grp)
    lines = []
    for k in range(n):
        deps, ins = mfmas[k]
        groups = [(tag, list(instrs)) for tag, instrs in slots[k]]
        if groups and groups[0][1] and groups[0][1][0].startswith("s_add_u32 m0"):
            lines.append(groups[0][1].pop(0))
        w = lds.wait_for(deps)
        if w is not None:
            lines.append("s_waitcnt lgkmcnt(%d)" % w)
        lines.append(ins)
        for tag, instrs in groups:
            lines.extend(instrs)
            if tag is not None:
                lds.issue(tag, sum(1 for x in instrs if x.startswith("ds_read")))
    for ins in m0_gaps(lines):
        e(ins)


def gen_main(v, e, L):
    """Prologue and K loop: K tiles of 64 through two (256-row tile) or three LDS buffers."""
    sT = S_T
    # temporaries
    s_kt, s_t1 = sT + 0, sT + 1
    s_ka1, s_kb1 = sT + 2, sT + 3       # K offsets of tile kt + 1
    s_ka2, s_kb2 = sT + 4, sT + 5       # K offsets of tile kt + 2
    s_tail1, s_oob1 = sT + 6, sT + 8    # pairs
    s_tail2, s_oob2 = sT + 10, sT + 12
    s_last = sT + 14                    # nk - 1
    s_zero = sT + 15
    s_waveA, s_waveB = sT + 20, sT + 21
    s_tmask, s_kta, s_ktb = sT + 22, sT + 24, sT + 25   # L2 prefetch: "K tile exists" mask (pair), its K offsets

    def tile_masks(s_tile, s_tail, s_oob):
        # tail mask: tile == nk - 1 ; oob mask: tile >= nk
        e("s_cmp_eq_u32 %s, %s" % (sr(s_tile), sr(s_last)))
        e("s_cselect_b64 %s, -1, 0" % sr(s_tail, 2))
        e("s_cmp_ge_u32 %s, %s" % (sr(s_tile), sr(S_NK)))
        e("s_cselect_b64 %s, -1, 0" % sr(s_oob, 2))

    # ------------------------------------------------------------------ prologue
    e("; ---- prologue (%s)" % v.name)
    e("v_mov_b32 %s, 0x80000000" % vr(V_OOB))
    # s[S_SPARE] = wave id | fix-up flags << 8 (bit 0: first chunk of the k range is partial, bit 1: last chunk)
    s_flags = sT + 18
    e("s_lshr_b32 %s, %s, 8" % (sr(s_flags), sr(S_SPARE)))
    e("s_and_b32 %s, %s, 0xff" % (sr(sT + 19), sr(S_SPARE)))
    e("s_sub_u32 %s, %s, 1" % (sr(s_last), sr(S_NK)))
    e("s_mov_b32 %s, 0" % sr(s_zero))
    # wave part of the LDS copy destinations: wave id is in s[S_SPARE]
    e("s_mul_i32 %s, %s, %d" % (sr(s_waveA), sr(sT + 19), v.na * (TR_BLOCK if v.a_tr else 1024)))
    e("s_add_u32 %s, %s, %s" % (sr(s_waveA), sr(s_waveA), sr(S_LDS)))
    e("s_mul_i32 %s, %s, %d" % (sr(s_waveB), sr(sT + 19), v.nb * (TR_BLOCK if v.b_tr else 1024)))
    e("s_add_u32 %s, %s, %s" % (sr(s_waveB), sr(s_waveB), sr(S_LDS)))
    # tile 0 -> buffer 0 (head offsets)
    for n in range(v.ncopy):
        for ins in m0_gaps(v.dma(n, 0, "head", 0, 0, s_zero, s_zero, V_TMP)):
            e(ins)
    S = v.stages
    c3, c0, c1, c2 = v.sched
    if S == 3:
        # fragment read addresses per buffer (the wrapper passes those of buffer 0)
        for is_a in (True, False):
            tr = v.a_tr if is_a else v.b_tr
            stage = v.a_stage if is_a else v.b_stage
            src, dst = (V_RA, V_BUFA) if is_a else (V_RB, V_BUFB)
            for buf in range(S):
                for sp in range(1 if tr else 2):
                    e("v_add_u32 %s, %d, %s" % (vr(dst + 2 * buf + sp), buf * stage, vr(src + sp)))
    # tiles 1 .. S - 2 -> their buffers in full, tile S - 1 -> buffer S - 1: the first c3 copies
    slots = [(s_tail1, s_oob1, s_ka1, s_kb1), (s_tail2, s_oob2, s_ka2, s_kb2)]
    for tix in range(1, S):
        s_tail, s_oob, s_ka, s_kb = slots[tix - 1]
        e("s_mov_b32 %s, %d" % (sr(s_t1), tix))
        tile_masks(s_t1, s_tail, s_oob)
        e("s_mul_i32 %s, %s, %d" % (sr(s_ka), sr(S_ASTEP), tix))
        e("s_mul_i32 %s, %s, %d" % (sr(s_kb), sr(S_BSTEP), tix))
        for n in range(v.ncopy if tix < S - 1 else c3):
            for ins in m0_gaps(v.dma(n, tix, "loop", s_tail, s_oob, s_ka, s_kb, V_TMP + (n % 8))):
                e(ins)
    # L2 prefetch of the K tiles that the loop's touches (tile kt + TOUCH_DIST) do not reach
    n_pro_touch = 0
    if v.nt:
        for tix in range(S, v.touch_dist):
            e("s_cmp_gt_u32 %s, %d" % (sr(S_NK), tix))
            e("s_cselect_b64 %s, -1, 0" % sr(s_tmask, 2))
            e("s_mul_i32 %s, %s, %d" % (sr(s_kta), sr(S_ASTEP), tix))
            e("s_mul_i32 %s, %s, %d" % (sr(s_ktb), sr(S_BSTEP), tix))
            for k, op in enumerate(v.touch):
                for ins in touch_group(v, op, s_tmask, s_kta if op == "a" else s_ktb, V_TMP + 8 + k):
                    e(ins)
                n_pro_touch += 1
    # zero the accumulators while the copies fly
    for r in range(64 * v.tm):
        e("v_accvgpr_write_b32 a%d, 0" % r)
    e("s_waitcnt vmcnt(%d)" % ((S - 2) * v.ncopy + c3 + n_pro_touch))
    e("s_barrier")
    has_kc = not (v.a_tr and v.b_tr)
    if has_kc:
        # partial first / last chunk of a jagged k range (tile 0 is also the last tile when nk == 1)
        e("s_and_b32 %s, %s, 3" % (sr(s_t1), sr(s_flags)))
        e("s_cmp_eq_u32 %s, 0" % sr(s_t1))
        e("s_cbranch_scc1 L_nofix0_%s" % L)
        e("s_bitcmp1_b32 %s, 0" % sr(s_flags))
        e("s_cbranch_scc0 L_nohead_%s" % L)
        fixup(e, v, 0, 0)
        e("s_waitcnt lgkmcnt(0)")
        e.label("L_nohead_%s" % L)
        e("s_bitcmp1_b32 %s, 1" % sr(s_flags))
        e("s_cbranch_scc0 L_notail0_%s" % L)
        e("s_cmp_eq_u32 %s, 1" % sr(S_NK))
        e("s_cbranch_scc0 L_notail0_%s" % L)
        fixup(e, v, 1, 0)
        e.label("L_notail0_%s" % L)
        e("s_waitcnt lgkmcnt(0)")
        e("s_barrier")
        e.label("L_nofix0_%s" % L)
    for tag, instrs in v.first_reads(0):
        for ins in instrs:
            e(ins)
    e("s_mov_b32 %s, 0" % sr(s_kt))
    e("s_cmp_eq_u32 %s, 0" % sr(S_NK))
    e("s_cbranch_scc1 L_done_%s" % L)

    # ------------------------------------------------------------------ K loop, two tiles per trip
    def tagged(groups):
        return [(None, g) for g in groups]

    def mix(reads, others):
        """Both lists spread over the whole step, each keeping its order: the four waves of a workgroup issue
        their copies at the same time, and bunched up they ask more of the address unit than it takes."""
        keyed = [((i + 0.5) / len(reads), 0, i, g) for i, g in enumerate(reads)]
        keyed += [((j + 0.5) / len(others), 1, j, g) for j, g in enumerate(others)]
        return [g for _, _, _, g in sorted(keyed, key=lambda x: x[:3])]

    def ktile(buf, fast):
        # on entry: the fragments of step 0 are in flight (first_reads); the first c3 copies of tile kt + S - 1 too.
        # fast: tiles kt + S - 1 and kt + S are both before the last one, so their copies need neither the
        # tail offsets nor the out-of-range select, and tile kt + 1 cannot be the last one.
        which = "fast" if fast else "loop"
        e("; ---- k tile on buffer %d%s" % (buf, " (interior)" if fast else ""))
        lds = LdsOrder(tag for tag, instrs in v.first_reads(buf) for _ in instrs)
        # K offsets (and masks) of tiles kt + S - 1 (copied during steps 0..2) and kt + S (step 3)
        e("s_add_u32 %s, %s, %d" % (sr(s_t1), sr(s_kt), S - 1))
        if not fast:
            tile_masks(s_t1, s_tail1, s_oob1)
        e("s_mul_i32 %s, %s, %s" % (sr(s_ka1), sr(s_t1), sr(S_ASTEP)))
        e("s_mul_i32 %s, %s, %s" % (sr(s_kb1), sr(s_t1), sr(S_BSTEP)))
        e("s_add_u32 %s, %s, %d" % (sr(s_t1), sr(s_kt), S))
        if not fast:
            tile_masks(s_t1, s_tail2, s_oob2)
        e("s_mul_i32 %s, %s, %s" % (sr(s_ka2), sr(s_t1), sr(S_ASTEP)))
        e("s_mul_i32 %s, %s, %s" % (sr(s_kb2), sr(s_t1), sr(S_BSTEP)))
        if v.nt:
            e("s_add_u32 %s, %s, %d" % (sr(s_t1), sr(s_kt), v.touch_dist))
            e("s_cmp_lt_u32 %s, %s" % (sr(s_t1), sr(S_NK)))
            e("s_cselect_b64 %s, -1, 0" % sr(s_tmask, 2))
            e("s_mul_i32 %s, %s, %s" % (sr(s_kta), sr(s_t1), sr(S_ASTEP)))
            e("s_mul_i32 %s, %s, %s" % (sr(s_ktb), sr(s_t1), sr(S_BSTEP)))
        nb = (buf + 1) % S       # buffer of tile kt + 1
        cb = (buf + S - 1) % S   # buffer of tile kt + S - 1
        # step 0: the reads of step 1 (and half of the B fragments of k 32..63), next copies of tile kt + S - 1
        side = mix(v.step_reads(0, buf, nb),
                   tagged(v.dma(n, cb, which, s_tail1, s_oob1, s_ka1, s_kb1, V_TMP + (n % 8)) for n in range(c3, c3 + c0)))
        interleave(e, lds, v.mfmas(0), side)
        # step 1
        side = mix(v.step_reads(1, buf, nb),
                   tagged(v.dma(n, cb, which, s_tail1, s_oob1, s_ka1, s_kb1, V_TMP + (n % 8)) for n in range(c3 + c0, c3 + c0 + c1)))
        interleave(e, lds, v.mfmas(1), side)
        # step 2
        side = mix(v.step_reads(2, buf, nb),
                   tagged(v.dma(n, cb, which, s_tail1, s_oob1, s_ka1, s_kb1, V_TMP + (n % 8)) for n in range(c3 + c0 + c1, v.ncopy)))
        # the touches come after every copy of tile kt + S - 1 in issue order, so the wait below can leave them
        # in flight: they have until the next K tile's wait to land
        side += tagged(touch_group(v, op, s_tmask, s_kta if op == "a" else s_ktb, V_TMP + 8 + k) for k, op in enumerate(v.touch))
        interleave(e, lds, v.mfmas(2), side)
        # tile kt+1 has landed for this wave; after the barrier for all, and `buf` is free
        e("s_waitcnt vmcnt(%d) lgkmcnt(0)" % ((S - 2) * (v.ncopy + v.nt) + v.nt))
        lds.clear()
        e("s_barrier")
        if not (v.a_tr and v.b_tr) and not fast:
            # the tile that has just landed is the last one and its last chunk is partial
            e("s_add_u32 %s, %s, 1" % (sr(s_t1), sr(s_kt)))
            e("s_cmp_eq_u32 %s, %s" % (sr(s_t1), sr(s_last)))
            e("s_cbranch_scc0 L_nofix%d_%s" % (buf + 1, L))
            e("s_bitcmp1_b32 %s, 1" % sr(sT + 18))
            e("s_cbranch_scc0 L_nofix%d_%s" % (buf + 1, L))
            fixup(e, v, 1, nb)
            e("s_waitcnt lgkmcnt(0)")
            e("s_barrier")
            e.label("L_nofix%d_%s" % (buf + 1, L))
        # step 3: the first fragments of the next tile, first copies of tile kt + S -> buf
        side = mix(v.step_reads(3, buf, nb),
                   tagged(v.dma(n, buf, which, s_tail2, s_oob2, s_ka2, s_kb2, V_TMP + (n % 8)) for n in range(0, c3)))
        interleave(e, lds, v.mfmas(3), side)
        e("s_add_u32 %s, %s, 1" % (sr(s_kt), sr(s_kt)))

    def ktile_both(buf):
        e("s_add_u32 %s, %s, %d" % (sr(s_t1), sr(s_kt), S))
        e("s_cmp_lt_u32 %s, %s" % (sr(s_t1), sr(s_last)))
        e("s_cbranch_scc0 L_slow%d_%s" % (buf, L))
        ktile(buf, True)
        e("s_branch L_join%d_%s" % (buf, L))
        e.label("L_slow%d_%s" % (buf, L))
        ktile(buf, False)
        e.label("L_join%d_%s" % (buf, L))

    e.label("L_loop_%s" % L)
    for buf in range(S - 1):
        ktile_both(buf)
        e("s_cmp_ge_u32 %s, %s" % (sr(s_kt), sr(S_NK)))
        e("s_cbranch_scc1 L_done_%s" % L)
    ktile_both(S - 1)
    e("s_cmp_lt_u32 %s, %s" % (sr(s_kt), sr(S_NK)))
    e("s_cbranch_scc1 L_loop_%s" % L)
    e.label("L_done_%s" % L)


def gen_variant(v):
    e = Emit()
    L = "%s_%%=" % v.name  # unique label suffix per asm instance
    gen_main(v, e, L)
    gen_epilogue(v, e, L)
    return e


def gen_epilogue(v, e, L):
    """Accumulators -> output.  The MFMA operands are swapped, so a lane owns 4 consecutive columns of a
    row: acc block (i, j), register r  ->  C[m = 16 i + lane % 16][n = 16 j + 4 (lane / 16) + r].
    The wave stages its block in LDS (rows padded to `pitch` bytes; `ipp` groups of 32 rows per pass: two for a
    16-bit output, one for fp32, whose rows are twice as long) and reads it back so that each lane
    holds 16 consecutive bytes of a row: every store instruction writes whole rows of the wave's 128 columns
    (256 contiguous bytes of 4 rows, or 512 contiguous bytes of 2 rows for fp32).
    v[V_EPI + 0] = stage write address, v[V_EPI + 1] = stage read address,
    v[V_EPI + 2] = store offset of the lane's chunk in read-back instruction 0 (or out-of-range when the
                   lane's columns are not all valid), v[V_EPI + 3] = its row - row_lo, valid iff (unsigned) < S_ROWCNT,
    v[V_EPI2 + 0] = that store offset whatever the validity, v[V_EPI2 + 1] = mask of valid elements of a
                   chunk that a group boundary cuts (tile flag bit 2): those go out element by element."""
    e("; ---- epilogue")
    e("s_waitcnt vmcnt(0) lgkmcnt(0)")
    e("s_nop 15")
    e("s_nop 15")
    e("s_barrier")
    t = 0                                 # temporaries of the epilogue: the fragment registers
    f32 = v.out_f32
    esz = 4 if f32 else 2
    nel = 16 // esz                       # elements of a 16-byte chunk
    pitch = PITCH32 if f32 else (PITCH_ACT if v.act else PITCH)
    # groups of 32 rows (two MFMA block rows) per pass: one for fp32 (its rows are twice as long), two for a 16-bit
    # output -- staged in one pass of 128 rows, the first store of a tile left 0.3 us later (batched workload
    # 1 to 3 % slower, the others the same)
    ipp = 1 if f32 else min(2, v.tm)
    ncol = 64 if v.act else 16 * v.tn     # elements of a staged row
    rpi = 1024 // (ncol * esz)            # rows per read-back instruction (64 lanes x 16 bytes)
    depth = 4
    regs = [t + 4 * x for x in range(depth)]          # read-back data, 4 registers each
    voff, vrow, vsel = t + 24, t + 25, t + 26
    eoff, vpoff, vtmp = t + 27, t + 35, t + 36
    e("v_mov_b32 %s, %s" % (vr(voff), vr(V_EPI + 2)))
    e("v_mov_b32 %s, %s" % (vr(vrow), vr(V_EPI + 3)))
    # eoff[el] = byte offset of element el of the lane's chunk if it is valid, else the out-of-range offset
    e("s_bitcmp1_b32 %s, 2" % sr(S_T + 18))
    e("s_cbranch_scc0 L_nopart_setup_%s" % L)
    e("v_mov_b32 %s, %s" % (vr(vpoff), vr(V_EPI2)))
    for el in range(nel):
        e("v_bfe_u32 %s, %s, %d, 1" % (vr(vtmp), vr(V_EPI2 + 1), el))
        e("v_cmp_ne_u32 vcc, 0, %s" % vr(vtmp))
        e("v_mov_b32 %s, %d" % (vr(vtmp), esz * el))
        e("v_cndmask_b32 %s, %s, %s, vcc" % (vr(eoff + el), vr(V_OOB), vr(vtmp)))
    e.label("L_nopart_setup_%s" % L)
    nstore = 0
    for p0 in range(0, v.tm, ipp):
        k = 0
        for il2 in range(2 * min(ipp, v.tm - p0)):
            i = 2 * p0 + il2                   # MFMA block row of the wave
            rowoff = 16 * il2 * pitch          # its first row in the staging area
            if v.act:
                # silu(g) * u = g * u / (1 + 2^(-g log2 e)); gate block j pairs with block j + 4 (64 columns on).
                # Four elements advance together, so no result of a transcendental is read by the next instruction.
                for j in range(4):
                    b = t + 12 * (k % 2)
                    k += 1
                    g0, u0 = v.acc(i, j), v.acc(i, j + 4)
                    for r in range(4):
                        e("v_accvgpr_read_b32 %s, a%d" % (vr(b + r), g0 + r))
                    for r in range(4):
                        e("v_accvgpr_read_b32 %s, a%d" % (vr(b + 4 + r), u0 + r))
                    for r in range(4):
                        e("v_mul_f32 %s, 0xbfb8aa3b, %s" % (vr(b + 8 + r), vr(b + r)))
                    for r in range(4):
                        e("v_exp_f32 %s, %s" % (vr(b + 8 + r), vr(b + 8 + r)))
                    e("s_nop 0")
                    for r in range(4):
                        e("v_add_f32 %s, 1.0, %s" % (vr(b + 8 + r), vr(b + 8 + r)))
                    for r in range(4):
                        e("v_rcp_f32 %s, %s" % (vr(b + 8 + r), vr(b + 8 + r)))
                    for r in range(4):
                        e("v_mul_f32 %s, %s, %s" % (vr(b + r), vr(b + r), vr(b + 4 + r)))
                    for r in range(4):
                        e("v_mul_f32 %s, %s, %s" % (vr(b + r), vr(b + r), vr(b + 8 + r)))
                    e("v_cvt_pk_%s_f32 %s, %s, %s" % (v.dt, vr(b + 8), vr(b), vr(b + 1)))
                    e("v_cvt_pk_%s_f32 %s, %s, %s" % (v.dt, vr(b + 9), vr(b + 2), vr(b + 3)))
                    e("ds_write_b64 %s, %s offset:%d" % (vr(V_EPI), vr(b + 8, 2), rowoff + 16 * j * 2))
                continue
            for j in range(v.tn):
                b = t + 6 * (k % 4)
                k += 1
                a0 = v.acc(i, j)
                for r in range(4):
                    e("v_accvgpr_read_b32 %s, a%d" % (vr(b + r), a0 + r))
                if f32:
                    e("ds_write_b128 %s, %s offset:%d" % (vr(V_EPI), vr(b, 4), rowoff + 16 * j * 4))
                else:
                    e("v_cvt_pk_%s_f32 %s, %s, %s" % (v.dt, vr(b + 4), vr(b), vr(b + 1)))
                    e("v_cvt_pk_%s_f32 %s, %s, %s" % (v.dt, vr(b + 5), vr(b + 2), vr(b + 3)))
                    e("ds_write_b64 %s, %s offset:%d" % (vr(V_EPI), vr(b + 4, 2), rowoff + 16 * j * 2))
        e("s_waitcnt lgkmcnt(0)")
        nrb = min(ipp, v.tm - p0) * 32 // rpi   # read-back instructions of this pass
        for r in range(min(depth, nrb)):
            e("ds_read_b128 %s, %s offset:%d" % (vr(regs[r], 4), vr(V_EPI + 1), r * rpi * pitch))
        for r in range(nrb):
            e("s_waitcnt lgkmcnt(%d)" % min(depth - 1, nrb - 1 - r))
            e("v_cmp_gt_u32 vcc, %s, %s" % (sr(S_ROWCNT), vr(vrow)))
            e("v_cndmask_b32 %s, %s, %s, vcc" % (vr(vsel), vr(V_OOB), vr(voff)))
            # non-temporal: the output is written once and not read by this kernel; kept out of the way, it does
            # not push operand panels that other workgroups are about to share out of the L2
            # a partial tile is read by the workgroup that adds the parts up, maybe on another XCD: written through
            # at device scope
            e("buffer_store_dwordx4 %s, %s, %s, 0 offen %s" % (vr(regs[r % depth], 4), vr(vsel), sr(S_RC, 4), "sc1" if v.partial else "nt"))
            e("s_bitcmp1_b32 %s, 2" % sr(S_T + 18))
            e("s_cbranch_scc0 L_nopart%d_%s" % (nstore, L))
            for el in range(nel):
                e("v_add_u32 %s, %s, %s" % (vr(vtmp), vr(eoff + el), vr(vpoff)))
                e("v_cndmask_b32 %s, %s, %s, vcc" % (vr(vtmp + 1 + el % 2), vr(V_OOB), vr(vtmp)))
                if f32:
                    e("buffer_store_dword %s, %s, %s, 0 offen" % (vr(regs[r % depth] + el), vr(vtmp + 1 + el % 2), sr(S_RC, 4)))
                else:
                    e("buffer_store_short%s %s, %s, %s, 0 offen" % ("_d16_hi" if el % 2 else "", vr(regs[r % depth] + el // 2),
                                                                     vr(vtmp + 1 + el % 2), sr(S_RC, 4)))
            e("v_add_u32 %s, %s, %s" % (vr(vpoff), sr(S_CSTEP), vr(vpoff)))
            e.label("L_nopart%d_%s" % (nstore, L))
            nstore += 1
            if r + depth < nrb:
                # the store above must have read its data before the register is reloaded
                e("s_nop 0")
                e("ds_read_b128 %s, %s offset:%d" % (vr(regs[r % depth], 4), vr(V_EPI + 1), (r + depth) * rpi * pitch))
            e("v_add_u32 %s, %s, %s" % (vr(voff), sr(S_CSTEP), vr(voff)))
            e("v_add_u32 %s, %d, %s" % (vr(vrow), rpi, vr(vrow)))
        if p0 + ipp < v.tm:
            # the next pass overwrites the staging area and the read-back registers: reads are done
            # (lgkmcnt 0 above); the last stores must have fetched their data
            e("s_nop 4")
    e("s_waitcnt lgkmcnt(0)")
    e("s_barrier")


def clobbers(v):
    c = ["memory", "vcc", "scc"]
    c += ["v%d" % i for i in range(0, V_CLOBBER)] + ["v%d" % V_OOB]
    c += ["a%d" % i for i in range(256)]
    c += ["s%d" % i for i in range(S_T, S_T + 34)]
    return ", ".join('"%s"' % x for x in c)


def main():
    out = []
    out.append("// Generated by gen_tile_asm.py -- do not edit.")
    out.append("// Per-tile main loop + epilogue in gfx950 assembly, one function per operand-layout / output variant.")
    out.append("#define GMM_TILE_PITCH %d" % PITCH)
    out.append("#define GMM_TILE_PITCH32 %d" % PITCH32)
    out.append("#define GMM_TILE_TR_BLOCK %d" % TR_BLOCK)
    out.append("#define GMM_TILE_KC_STAGE %d" % KC_STAGE)
    out.append("#define GMM_TILE_TR_STAGE %d" % TR_STAGE)
    out.append("#define GMM_TILE_STAGING_BYTES %d" % STAGE_BYTES)
    out.append("#define GMM_TILE_STAGES_SHORT %d" % STAGES_SHORT)
    out.append("#define GMM_TILE_PITCH_ACT %d" % PITCH_ACT)
    for f16 in (0, 1):
        for a_tr, b_tr, f32, tm, b_nt, act in [(a, b, f, t, n, c) for a in (0, 1) for b in (0, 1) for f in (0, 1) for t in (4, 2, 1)
                                               for n in (0, 1) for c in (0, 1, 2)]:
            if tm != 4 and a_tr:
                continue
            if b_nt and tm == 4:
                continue      # only remainder tiles can be the sole reader of a B panel often enough to matter
            if act == 1 and (a_tr or f32):
                continue      # the gated epilogue: K-contiguous first operand, 16-bit output
            if act == 2 and (not f32 or b_nt):
                continue      # partial tiles: fp32, ordinary B copies
            v = Variant(a_tr, b_tr, f32, tm, f16, b_nt, act)
            e = gen_variant(v)
            out.append("")
            out.append("template <> __device__ __forceinline__ void gmm_tile_asm<%d, %d, %d, %d, %d, %d, %d>(GmmTileRegs& r) {" % (a_tr, b_tr, f32, tm, f16, b_nt, act))
            out.append("  asm volatile(")
            out.append(e.text())
            out.append("      :")
            pins = [(V_VOA_HEAD, 8, "voa_head"), (V_VOB_HEAD, 8, "vob_head"), (V_VOA, 8, "voa"), (V_VOB, 8, "vob"),
                    (V_VOA_TAIL, 8, "voa_tail"), (V_VOB_TAIL, 8, "vob_tail"), (V_RA, 4, "ra_addr"), (V_RB, 4, "rb_addr"),
                    (V_EPI, 4, "epi"), (V_EPI2, 2, "epi2"), (V_TOUCH, 2, "touch"), (V_FIX, 4, "fix")]
            out.append("      : " + ", ".join('"{v[%d:%d]}"(r.%s)' % (b0, b0 + n - 1, name) for b0, n, name in pins) + ",")
            out.append('        "{s[28:35]}"(r.masks), "{s[36:39]}"(r.rsrc_a), "{s[40:43]}"(r.rsrc_b), "{s[44:47]}"(r.rsrc_c), "{s[48:55]}"(r.scal)')
            out.append("      : %s);" % clobbers(v))
            out.append("}")
    sys.stdout.write("\n".join(out) + "\n")


if __name__ == "__main__":
    main()
