#!/usr/bin/env python3
"""Generates the hand-scheduled main loops (gfx950 ISA, each one inline-asm
string) of the bf16 GEMM macro tiles:

    python gen_gemm_asm.py      > gemm_bf16_256_loop.inc        # 256 x 256, one workgroup per CU
    python gen_gemm_asm.py half > gemm_bf16_256x128_loop.inc    # 256 x 128, two per CU (end of file)
    python gen_gemm_asm.py quarter > gemm_bf16_128_loop.inc     # 128 x 128, three per CU (end of file)
    python gen_gemm_asm.py deep > gemm_bf16_256x128_deep_loop.inc  # 256 x 128, one per CU, the 256 x 256 pipeline

The rest of this comment describes the 256 x 256 loop.

Why hand-scheduled: with 256 accumulator registers per lane a SIMD holds one
wave, so nothing but instruction order hides LDS and memory latency.

Pipeline.  K is consumed in half-steps of 32 bf16 (64 bytes per tile row).  LDS
holds four stages of 32 KiB (W tile 256 rows x 64 B, then X tile); the tile of
half-step h lives in stage h % 4.  During half-step h a wave
  * issues 32 MFMAs (32x32x16): k-phase 0 on fragment set A, k-phase 1 on set B,
  * reads the k-phase-1 fragments of tile h (into B) behind the first MFMAs of
    phase 0 and the k-phase-0 fragments of tile h+1 (into A) behind the first
    MFMAs of phase 1, so no fragment read is ever waited for right after issue,
  * issues its 8 global->LDS loads of tile h+3 (three half-steps ahead, which
    keeps a steady stream of requests in flight instead of one burst per step),
  * ends with "s_waitcnt vmcnt(8)" -- everything but the 8 loads just issued,
    i.e. tile h+2, has landed -- and one s_barrier.
The barrier at the end of half-step h-1 therefore guarantees tile h+1, which is
what lets half-step h prefetch tile h+1's fragments before its own barrier.

Register plan (per lane):
  a[0:255]    accumulators: 4x4 blocks of 32x32 (inline-asm "+a" operands)
  v[112:127]  W fragments, set A (block i at 112+4i)   v[128:143]  X fragments, set A
  v[144:159]  W fragments, set B                       v[160:175]  X fragments, set B
  v[96:99]    LDS byte addresses of my fragment row in stage 0: W k-phase 0, W k-phase 1,
              X k-phase 0, X k-phase 1                 v[100:103]  the same + 65536 (stages 2, 3)
  v[104:107]  global lane offsets of my 4 W row groups v[108:111]  same for X
  (the registers above v175 stay free: with 256 accumulators the wave then leaves room on its
  SIMD for waves of small kernels from another stream)
  s96 / s98 K byte offset of the W / X tile being fetched, s97 loop counter,
  s92..s95    M0 base of stage 0..3 (stage base + wave * 1024)

LDS swizzle: a tile row is 64 bytes = four 16-byte chunks; chunk c of row r sits
in slot c ^ ((r >> 2) & 3), which spreads the fragment reads of any
8 or 16 consecutive rows over all banks.  One buffer_load_dwordx4 ... lds moves
16 rows (64 lanes x 16 B) to M0 + 16 * lane; the swizzle is applied on the
global side (which chunk a lane fetches).
"""
def vreg4(base):
    return "v[%d:%d]" % (base, base + 3)


class Emitter:
    def __init__(self):
        self.lines = []
        self.issued = 0            # LDS reads issued so far (monotonic)
        self.index = {}            # fragment register base -> issue index of its latest read
        self.guaranteed = None     # an upper bound on outstanding LDS reads already waited for

    def emit(self, text):
        self.lines.append(text)

    def read(self, dst, addr_reg, offset):
        assert 0 <= offset < 65536
        self.emit("ds_read_b128 %s, v%d offset:%d" % (vreg4(dst), addr_reg, offset))
        self.index[dst] = self.issued
        self.issued += 1
        if self.guaranteed is not None:
            self.guaranteed += 1

    def need(self, *regs):
        """Weakest s_waitcnt that guarantees the reads into `regs` have returned
        (LDS reads return in order)."""
        newest = max(self.index[r] for r in regs)
        allowed = self.issued - 1 - newest
        if self.guaranteed is None or allowed < self.guaranteed:
            self.emit("s_waitcnt lgkmcnt(%d)" % min(allowed, 15))
            self.guaranteed = allowed

    def forget_bound(self):
        self.guaranteed = None


NSTAGE = 4
DMA_EVERY = 2         # one global->LDS load behind every second MFMA


class Deep:
    """Register and LDS plan of the four-stage loop described above, for a wave tile of nwb x nxb accumulator
    blocks (32 features x 32 tokens each).  The 256 x 256 kernel is 4 x 4; "deep" mode builds the 256 x 128 tile
    (4 x 2, end of file) the same way."""

    def __init__(self, name, nwb, nxb, wa, xa, wb, xb, addr, wvoff, xvoff, stage):
        self.name, self.nwb, self.nxb = name, nwb, nxb
        self.wa, self.xa, self.wb, self.xb = wa, xa, wb, xb
        self.addr, self.wvoff, self.xvoff, self.stage = addr, wvoff, xvoff, stage
        self.ndma = nwb + nxb            # global->LDS loads per tile and wave = fragment reads per k-phase
        # the pair the first MFMA needs first, then the other X fragments, then the other W fragments
        self.read_order = [("w", 0)] + [("x", b) for b in range(nxb)] + [("w", b) for b in range(1, nwb)]

    def frag_reads(self, stage, kk, wset, xset):
        bank, half = stage >> 1, stage & 1
        out = []
        for kind, b in self.read_order:
            if kind == "w":
                out.append((wset + 4 * b, self.addr + 4 * bank + kk, half * self.stage + b * 2048))
            else:
                out.append((xset + 4 * b, self.addr + 4 * bank + 2 + kk, half * self.stage + b * 2048))
        return out

    def dma_instrs(self, stage):
        """The global->LDS loads of one tile into `stage`: (M0 update, load)."""
        out = []
        for k in range(self.ndma):
            m0 = ("s_mov_b32 m0, s%d" % (92 + stage)) if k == 0 else "s_add_u32 m0, m0, 0x1000"
            if k < self.nwb:
                ld = "buffer_load_dwordx4 v%d, %%[wres], s96 offen lds" % (self.wvoff + k)
            else:
                ld = "buffer_load_dwordx4 v%d, %%[xres], s98 offen lds" % (self.xvoff + k - self.nwb)
            out.append((m0, ld))
        return out

    def half_step(self, e, stage, dma, prefetch_next, vmcnt, barrier):
        """One half-step on `stage`.  On entry the reads of set A (k-phase 0 of this
        tile) have been issued, in read_order, as the latest LDS reads."""
        e.emit("; ---- half-step on stage %d%s" % (stage, ", fetch into stage %d" % ((stage + 3) % NSTAGE) if dma else ""))
        dmas = self.dma_instrs((stage + 3) % NSTAGE) if dma else []
        per_phase = self.nwb * self.nxb
        for kk in range(2):
            wset, xset = (self.wa, self.xa) if kk == 0 else (self.wb, self.xb)
            if kk == 0:
                pending = self.frag_reads(stage, 1, self.wb, self.xb)
            else:
                pending = self.frag_reads((stage + 1) % NSTAGE, 0, self.wa, self.xa) if prefetch_next else []
            m = 0
            for i in range(self.nwb):
                for j in range(self.nxb):
                    e.need(wset + 4 * i, xset + 4 * j)
                    gm = per_phase * kk + m
                    d = gm // DMA_EVERY if (dmas and gm % DMA_EVERY == 0 and gm // DMA_EVERY < self.ndma) else None
                    if d is not None:
                        e.emit(dmas[d][0])      # M0 update in front of the MFMA: the MFMA is the
                    e.emit("v_mfma_f32_32x32x16_bf16 %%[c%d%d], %s, %s, %%[c%d%d]" %   # wait state before M0 is used
                           (i, j, vreg4(wset + 4 * i), vreg4(xset + 4 * j), i, j))
                    if d is not None:
                        e.emit(dmas[d][1])
                    # The destination set of these reads was last used by MFMAs of the
                    # previous k-phase, all of which have issued.
                    if m < len(pending):
                        e.read(*pending[m])
                    m += 1
        if vmcnt is not None:
            e.emit("s_waitcnt vmcnt(%d)" % vmcnt)
        if barrier:
            e.emit("s_barrier")


def advance_k(e):
    """Next half-step along K: +64 bytes in a row-major operand, +16 KiB (one block) in a packed one."""
    e.emit("s_add_u32 s96, s96, %[wkstep]")
    e.emit("s_add_u32 s98, s98, %[xkstep]")


FULL = Deep("", 4, 4, 112, 128, 144, 160, 96, 104, 108, 0x8000)
# "deep" mode: python gen_gemm_asm.py deep > gemm_bf16_256x128_deep_loop.inc
# The 256 x 128 tile (4 x 2 accumulator blocks per wave) with the pipeline of the 256 x 256 loop: four stages of
# 24 KiB (W tile at +0, X tile at +0x4000, which the kernel puts into %[xb]), loads three half-steps ahead, no
# fragment read waited for right after issue.  96 KiB of LDS: one workgroup per CU, which is what a launch of at
# most 256 workgroups gets anyway; there the two-per-CU loop ("half" mode) leaves the matrix pipe idle half of the
# time, because nothing runs beside it while it waits for the last fragment reads of a half-step and the barrier.
#   v64..v79 / v80..v87  W / X fragments, set A      v88..v103 / v104..v111  set B
#   v112..v119  fragment row addresses (stages 0-1, 2-3)   v120..v123 / v124..v125  W / X lane offsets
DEEP = Deep("deep", 4, 2, 64, 80, 88, 104, 112, 120, 124, 0x6000)


def main(c=FULL):
    e = Emitter()
    e.emit("; ======== setup ========")
    e.emit("v_mov_b32 v%d, %%[wb]" % (c.addr + 0))
    e.emit("v_xor_b32 v%d, 0x20, %%[wb]" % (c.addr + 1))
    e.emit("v_mov_b32 v%d, %%[xb]" % (c.addr + 2))
    e.emit("v_xor_b32 v%d, 0x20, %%[xb]" % (c.addr + 3))
    for r in range(4):
        e.emit("v_add_u32 v%d, 0x%x, v%d" % (c.addr + 4 + r, 2 * c.stage, c.addr + r))
    e.emit("v_mov_b32 v%d, %%[wv0]" % c.wvoff)
    e.emit("v_mov_b32 v%d, %%[xv0]" % c.xvoff)
    for i in range(1, max(c.nwb, c.nxb)):
        if i < c.nwb:
            e.emit("v_add_u32 v%d, %%[w64], v%d" % (c.wvoff + i, c.wvoff + i - 1))
        if i < c.nxb:
            e.emit("v_add_u32 v%d, %%[x64], v%d" % (c.xvoff + i, c.xvoff + i - 1))
    # zero the accumulators: 0 * 0 + 0 through the matrix pipe (the accumulator
    # operands are write-only for the compiler, which halves the operand count)
    for r in range(4):
        e.emit("v_mov_b32 v%d, 0" % (c.wa + r))
    e.emit("s_nop 7")      # VALU result -> MFMA source operand needs wait states the assembler does not add
    for i in range(c.nwb):
        for j in range(c.nxb):
            e.emit("v_mfma_f32_32x32x16_bf16 %%[c%d%d], %s, %s, 0" % (i, j, vreg4(c.wa), vreg4(c.wa)))
    e.emit("s_mov_b32 s92, %[m0b]")
    for s in range(1, NSTAGE):
        e.emit("s_add_u32 s%d, s%d, 0x%x" % (92 + s, 92 + s - 1, c.stage))
    e.emit("; ======== prologue: tiles 0, 1, 2 -> stages 0, 1, 2 ========")
    e.emit("s_mov_b32 s96, 0")
    e.emit("s_mov_b32 s98, 0")
    for t in range(3):
        for m0, ld in c.dma_instrs(t):
            e.emit(m0)
            e.emit("s_nop 0")
            e.emit(ld)
        if t < 2:
            advance_k(e)
    e.emit("s_waitcnt vmcnt(%d)" % c.ndma)          # tiles 0 and 1 have landed
    e.emit("s_barrier")
    for r in c.frag_reads(0, 0, c.wa, c.xa):
        e.read(*r)
    e.emit("s_mov_b32 s97, 4")
    e.emit("s_cmp_ge_u32 s97, %[ht]")
    e.emit("s_cbranch_scc1 L_tail_%=")
    e.emit("L_loop_%=:")
    for s in range(NSTAGE):
        advance_k(e)
        c.half_step(e, s, dma=True, prefetch_next=True, vmcnt=c.ndma, barrier=True)
    e.forget_bound()                       # the loop head is reached from two places
    e.emit("s_add_u32 s97, s97, 4")
    e.emit("s_cmp_lt_u32 s97, %[ht]")
    e.emit("s_cbranch_scc1 L_loop_%=")
    e.emit("L_tail_%=:")
    e.forget_bound()
    advance_k(e)
    c.half_step(e, 0, dma=True, prefetch_next=True, vmcnt=c.ndma, barrier=True)      # fetches the last tile
    c.half_step(e, 1, dma=False, prefetch_next=True, vmcnt=0, barrier=True)
    c.half_step(e, 2, dma=False, prefetch_next=True, vmcnt=None, barrier=False)
    c.half_step(e, 3, dma=False, prefetch_next=False, vmcnt=None, barrier=False)
    print("// Generated by gen_gemm_asm.py%s -- do not edit." % (" " + c.name if c.name else ""))
    for ln in e.lines:
        print('"%s\\n"' % ln)


# ---------------------------------------------------------------------------
# 256 x 128 macro tile, two workgroups per CU ("half" mode):
#     python gen_gemm_asm.py half > gemm_bf16_256x128_loop.inc
#
# A wave owns 128 features x 64 tokens = 4 x 2 accumulator blocks (128 AGPRs) and
# stays below 128 VGPRs, so a SIMD holds two waves of two different workgroups:
# while one workgroup is in its prologue or epilogue the other one's main loop
# has the matrix pipe.  Three LDS stages of 24 KiB (W tile 256 rows x 64 B at +0,
# X tile 128 rows x 64 B at +0x4000); the tile of half-step h lives in stage
# h % 3 and the loads of tile h+2 are issued during half-step h.  The loop body
# is ONE half-step; the stage rotates through scalar byte offsets, so any number
# of half-steps works and there is no separate tail:
#   s92  stage offset of the tile being multiplied      (0, 0x6000, 0xC000)
#   s93  stage offset of the tile being fetched
#   s94  M0 base (LDS base + wave * 1024)   s96 / s98  K byte offsets   s97  counter
#   v112..v115  fragment row addresses in stage 0: W k-phase 0, W k-phase 1, X k-phase 0, X k-phase 1
#   v122..v125  the same for the current stage      v116..v119 / v120..v121  W / X lane offsets
#   v64..v79 / v80..v87  W / X fragments, set A      v88..v103 / v104..v111  set B
# A half-step, skewed by one k-phase so that no fragment read is waited for right after
# issue: 6 reads of this tile's k-phase 0 (set A); 8 MFMAs on set B = the previous tile's
# k-phase 1, read a half-step ago; 8 MFMAs on A with the 6 reads of this tile's k-phase 1
# (into B) behind them; the 6 global->LDS loads of tile h+2 spread behind the MFMAs;
# vmcnt(6) (everything but the loads just issued, i.e. tile h+1, has landed); barrier.  Loads
# issued for tiles past the end of K fetch the last tile again and are never used; the
# block ends with vmcnt(0) and a barrier so that nothing lands in the LDS afterwards.
class Skewed:
    """Register and LDS plan of a loop whose body is one skewed half-step (see above): `nw` accumulator block
    rows (32 features each) per wave; two block columns (64 tokens)."""

    def __init__(self, name, nw, wa, xa, wb, xb, base, cur, wvoff, xvoff, x_lds, stage, nstage=3):
        self.name, self.nw, self.nstage = name, nw, nstage
        self.wa, self.xa, self.wb, self.xb = wa, xa, wb, xb
        self.base, self.cur, self.wvoff, self.xvoff = base, cur, wvoff, xvoff
        self.x_lds, self.stage = x_lds, stage
        self.n = nw + 2            # fragment reads per k-phase = global->LDS loads per tile and wave


HALF = Skewed("half", 4, 64, 80, 88, 104, 112, 122, 116, 120, 0x4000, 0x6000)
# 128 x 128 macro tile, three workgroups per CU ("quarter" mode):
#     python gen_gemm_asm.py quarter > gemm_bf16_128_loop.inc
# The same loop with a W tile of 128 rows: a wave owns 64 features x 64 tokens = 2 x 2 accumulator blocks
# (64 AGPRs) and everything the block writes lies below v92, so a SIMD holds three waves of three
# workgroups; three LDS stages of 16 KiB (W tile at +0, X tile at +0x2000).  Per half-step a wave issues
# 8 MFMAs, 8 fragment reads and 4 global->LDS loads.  For problems too small to fill the chip with the
# larger tiles.  The K offsets start at %[wk0] / %[xk0] (split K: a workgroup's share of K).
#   v48..v55 / v56..v63  W / X fragments, set A      v64..v71 / v72..v79  set B
#   v80..v83  fragment row addresses in stage 0      v84..v87  the same for the current stage
#   v88..v89 / v90..v91  W / X lane offsets
QUARTER = Skewed("quarter", 2, 48, 56, 64, 72, 80, 84, 88, 90, 0x2000, 0x4000)


def main_skewed(c):
    quarter = c.name == "quarter"
    e = Emitter()
    e.emit("; ======== setup ========")
    e.emit("v_mov_b32 v%d, %%[wb]" % (c.base + 0))
    e.emit("v_xor_b32 v%d, 0x20, %%[wb]" % (c.base + 1))
    e.emit("v_mov_b32 v%d, %%[xb]" % (c.base + 2))
    e.emit("v_xor_b32 v%d, 0x20, %%[xb]" % (c.base + 3))
    e.emit("v_mov_b32 v%d, %%[wv0]" % c.wvoff)
    e.emit("v_mov_b32 v%d, %%[xv0]" % c.xvoff)
    for i in range(1, c.nw):
        e.emit("v_add_u32 v%d, %%[w64], v%d" % (c.wvoff + i, c.wvoff + i - 1))
    e.emit("v_add_u32 v%d, %%[x64], v%d" % (c.xvoff + 1, c.xvoff))
    for r in range(4):
        e.emit("v_mov_b32 v%d, 0" % (c.wa + r))
    e.emit("s_nop 7")      # VALU result -> MFMA source operand
    for i in range(c.nw):
        for j in range(2):
            e.emit("v_mfma_f32_32x32x16_bf16 %%[c%d%d], %s, %s, 0" % (i, j, vreg4(c.wa), vreg4(c.wa)))
    e.emit("s_mov_b32 s94, %[m0b]")
    e.emit("s_mov_b32 s92, 0")
    e.emit("s_mov_b32 s93, 0")
    e.emit("s_mov_b32 s96, %s" % ("%[wk0]" if quarter else "0"))
    e.emit("s_mov_b32 s98, %s" % ("%[xk0]" if quarter else "0"))

    def dma(k):
        """k-th of the wave's loads of the tile at stage offset s93: (M0 update, load)."""
        m0 = "s_add_u32 m0, s94, s93" if k == 0 else "s_add_u32 m0, m0, 0x1000"
        if k < c.nw:
            ld = "buffer_load_dwordx4 v%d, %%[wres], s96 offen lds" % (c.wvoff + k)
        else:
            ld = "buffer_load_dwordx4 v%d, %%[xres], s98 offen lds" % (c.xvoff + k - c.nw)
        return m0, ld

    def rotate(reg):
        e.emit("s_add_u32 s%d, s%d, 0x%x" % (reg, reg, c.stage))
        e.emit("s_cmp_eq_u32 s%d, 0x%x" % (reg, c.nstage * c.stage))
        e.emit("s_cselect_b32 s%d, 0, s%d" % (reg, reg))

    e.emit("; ======== prologue: tiles 0, 1 -> stages 0, 1 ========" if c.nstage == 3 else
           "; ======== prologue: tiles 0 .. %d -> stages 0 .. %d ========" % (c.nstage - 2, c.nstage - 2))
    ahead = c.n * (c.nstage - 2)      # loads of the tiles that need not have landed when a half-step ends
    def advance_k_clamped():
        # The loads run two tiles ahead of the multiply, so the last two half-steps ask for tiles
        # past the end of K: they fetch the last tile again (the range check of a buffer
        # descriptor does not cover the scalar offset, so the offset itself has to stay inside).
        advance_k(e)
        e.emit("s_min_u32 s96, s96, %[wkmax]")
        e.emit("s_min_u32 s98, s98, %[xkmax]")

    for t in range(c.nstage - 1):
        for k in range(c.n):
            m0, ld = dma(k)
            e.emit(m0)
            e.emit("s_nop 0")
            e.emit(ld)
        rotate(93)
        advance_k_clamped()
    e.emit("s_waitcnt vmcnt(%d)" % ahead)         # tile 0 has landed
    e.emit("s_barrier")

    def reads(kk, wset, xset):
        out = [(wset + 4 * b, c.cur + kk, b * 2048) for b in range(c.nw)]
        out += [(xset + 4 * b, c.cur + 2 + kk, c.x_lds + b * 2048) for b in range(2)]
        # first the pair the first MFMA needs
        return [out[0], out[c.nw], out[c.nw + 1]] + out[1:c.nw]

    def cur_addresses():
        for r in range(4):
            e.emit("v_add_u32 v%d, s92, v%d" % (c.cur + r, c.base + r))

    def mfmas(wset, xset, tracked, pending, dma_from):
        """The MFMAs on one fragment set; `pending` LDS reads and half of the tile's DMA loads, from
        number dma_from on, go behind them."""
        n_dma = 0
        m = 0
        for i in range(c.nw):
            for j in range(2):
                if tracked:
                    e.need(wset + 4 * i, xset + 4 * j)
                d = dma_from + n_dma if (dma_from is not None and m % 2 == 0 and n_dma < c.n // 2) else None
                if d is not None:
                    e.emit(dma(d)[0])
                e.emit("v_mfma_f32_32x32x16_bf16 %%[c%d%d], %s, %s, %%[c%d%d]" %
                       (i, j, vreg4(wset + 4 * i), vreg4(xset + 4 * j), i, j))
                if d is not None:
                    e.emit(dma(d)[1])
                    n_dma += 1
                if m < len(pending):
                    e.read(*pending[m])
                m += 1

    def end_of_half_step():
        rotate(92)
        rotate(93)
        advance_k_clamped()
        # vmcnt(n): everything but the loads just issued, i.e. the next tile, has landed.
        # lgkmcnt(0): my reads of this tile are done before anybody may overwrite its stage.
        e.emit("s_waitcnt vmcnt(%d) lgkmcnt(0)" % ahead)
        e.emit("s_barrier")

    # The pipeline is skewed by one k-phase: a half-step starts by reading its tile's k-phase-0
    # fragments (set A) and multiplies the PREVIOUS tile's k-phase 1 (set B, read a half-step
    # ago) while they arrive; then k-phase 0 on set A while k-phase 1 is read into set B.
    e.emit("; ======== half-step 0: no previous tile ========")
    cur_addresses()
    for r in reads(0, c.wa, c.xa):
        e.read(*r)
    mfmas(c.wa, c.xa, True, reads(1, c.wb, c.xb), 0)
    # the remaining loads of tile 2 without MFMAs to hide behind
    for k in range(c.n // 2, c.n):
        e.emit(dma(k)[0])
        e.emit("s_nop 0")
        e.emit(dma(k)[1])
    end_of_half_step()
    e.emit("s_mov_b32 s97, 1")
    e.emit("s_cmp_ge_u32 s97, %[ht]")
    e.emit("s_cbranch_scc1 L_last_%=")
    e.emit("L_loop_%=:")
    cur_addresses()
    for r in reads(0, c.wa, c.xa):
        e.read(*r)
    e.emit("s_waitcnt lgkmcnt(%d)" % c.n)         # set B (read during the previous half-step) is complete
    e.forget_bound()
    e.guaranteed = c.n
    mfmas(c.wb, c.xb, False, [], 0)
    mfmas(c.wa, c.xa, True, reads(1, c.wb, c.xb), c.n // 2)
    end_of_half_step()
    e.emit("s_add_u32 s97, s97, 1")
    e.emit("s_cmp_lt_u32 s97, %[ht]")
    e.emit("s_cbranch_scc1 L_loop_%=")
    e.emit("L_last_%=:")
    e.emit("s_waitcnt lgkmcnt(0)")
    e.emit("; ======== k-phase 1 of the last tile ========")
    mfmas(c.wb, c.xb, False, [], None)
    e.emit("s_waitcnt vmcnt(0)")
    e.emit("s_barrier")
    print("// Generated by gen_gemm_asm.py %s -- do not edit." % c.name)
    for ln in e.lines:
        print('"%s\\n"' % ln)


if __name__ == "__main__":
    import sys
    if len(sys.argv) > 1 and sys.argv[1] == "half":
        if len(sys.argv) > 2:
            HALF.nstage = int(sys.argv[2])
        main_skewed(HALF)
    elif len(sys.argv) > 1 and sys.argv[1] == "deep":
        main(DEEP)
    elif len(sys.argv) > 1 and sys.argv[1] == "quarter":
        if len(sys.argv) > 2:
            QUARTER.nstage = int(sys.argv[2])
        main_skewed(QUARTER)
    else:
        main()
