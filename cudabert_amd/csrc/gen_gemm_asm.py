#!/usr/bin/env python3
"""Generates the hand-scheduled main loops (gfx950 ISA, each one inline-asm
string) of the bf16 GEMM macro tiles:

    python gen_gemm_asm.py      > gemm_bf16_256_loop.inc        # 256 x 256, one workgroup per CU
    python gen_gemm_asm.py half > gemm_bf16_256x128_loop.inc    # 256 x 128, two per CU (end of file)

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
WA, XA, WB, XB = 112, 128, 144, 160
ADDR = 96             # + 4 * bank + {0: W kk0, 1: W kk1, 2: X kk0, 3: X kk1}
W_VOFF, X_VOFF = 104, 108
NSTAGE = 4


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


READ_ORDER = [("w", 0), ("x", 0), ("x", 1), ("x", 2), ("x", 3), ("w", 1), ("w", 2), ("w", 3)]


def frag_reads(stage, kk, wset, xset):
    bank, half = stage >> 1, stage & 1
    out = []
    for kind, b in READ_ORDER:
        if kind == "w":
            out.append((wset + 4 * b, ADDR + 4 * bank + kk, half * 32768 + b * 2048))
        else:
            out.append((xset + 4 * b, ADDR + 4 * bank + 2 + kk, half * 32768 + b * 2048))
    return out


def dma_instrs(stage):
    """The eight global->LDS loads of one tile into `stage`: (M0 update, load)."""
    out = []
    for k in range(8):
        m0 = ("s_mov_b32 m0, s%d" % (92 + stage)) if k == 0 else "s_add_u32 m0, m0, 0x1000"
        if k < 4:
            ld = "buffer_load_dwordx4 v%d, %%[wres], s96 offen lds" % (W_VOFF + k)
        else:
            ld = "buffer_load_dwordx4 v%d, %%[xres], s98 offen lds" % (X_VOFF + k - 4)
        out.append((m0, ld))
    return out


DMA_EVERY = 2         # one global->LDS load behind every second MFMA


def half_step(e, stage, dma, prefetch_next, vmcnt, barrier):
    """One half-step on `stage`.  On entry the 8 reads of set A (k-phase 0 of this
    tile) have been issued, in READ_ORDER, as the latest 8 LDS reads."""
    e.emit("; ---- half-step on stage %d%s" % (stage, ", fetch into stage %d" % ((stage + 3) % NSTAGE) if dma else ""))
    dmas = dma_instrs((stage + 3) % NSTAGE) if dma else []
    for kk in range(2):
        wset, xset = (WA, XA) if kk == 0 else (WB, XB)
        if kk == 0:
            pending = frag_reads(stage, 1, WB, XB)
        else:
            pending = frag_reads((stage + 1) % NSTAGE, 0, WA, XA) if prefetch_next else []
        m = 0
        for i in range(4):
            for j in range(4):
                e.need(wset + 4 * i, xset + 4 * j)
                gm = 16 * kk + m
                d = gm // DMA_EVERY if (dmas and gm % DMA_EVERY == 0 and gm // DMA_EVERY < 8) else None
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


def main():
    e = Emitter()
    e.emit("; ======== setup ========")
    e.emit("v_mov_b32 v%d, %%[wb]" % (ADDR + 0))
    e.emit("v_xor_b32 v%d, 0x20, %%[wb]" % (ADDR + 1))
    e.emit("v_mov_b32 v%d, %%[xb]" % (ADDR + 2))
    e.emit("v_xor_b32 v%d, 0x20, %%[xb]" % (ADDR + 3))
    for r in range(4):
        e.emit("v_add_u32 v%d, 0x10000, v%d" % (ADDR + 4 + r, ADDR + r))
    e.emit("v_mov_b32 v%d, %%[wv0]" % W_VOFF)
    e.emit("v_mov_b32 v%d, %%[xv0]" % X_VOFF)
    for i in range(1, 4):
        e.emit("v_add_u32 v%d, %%[w64], v%d" % (W_VOFF + i, W_VOFF + i - 1))
        e.emit("v_add_u32 v%d, %%[x64], v%d" % (X_VOFF + i, X_VOFF + i - 1))
    # zero the accumulators: 0 * 0 + 0 through the matrix pipe (the accumulator
    # operands are write-only for the compiler, which halves the operand count)
    for r in range(4):
        e.emit("v_mov_b32 v%d, 0" % (WA + r))
    e.emit("s_nop 7")      # VALU result -> MFMA source operand needs wait states the assembler does not add
    for i in range(4):
        for j in range(4):
            e.emit("v_mfma_f32_32x32x16_bf16 %%[c%d%d], %s, %s, 0" % (i, j, vreg4(WA), vreg4(WA)))
    e.emit("s_mov_b32 s92, %[m0b]")
    for s in range(1, NSTAGE):
        e.emit("s_add_u32 s%d, s%d, 0x8000" % (92 + s, 92 + s - 1))
    e.emit("; ======== prologue: tiles 0, 1, 2 -> stages 0, 1, 2 ========")
    e.emit("s_mov_b32 s96, 0")
    e.emit("s_mov_b32 s98, 0")
    for t in range(3):
        for m0, ld in dma_instrs(t):
            e.emit(m0)
            e.emit("s_nop 0")
            e.emit(ld)
        if t < 2:
            advance_k(e)
    e.emit("s_waitcnt vmcnt(8)")          # tiles 0 and 1 have landed
    e.emit("s_barrier")
    for r in frag_reads(0, 0, WA, XA):
        e.read(*r)
    e.emit("s_mov_b32 s97, 4")
    e.emit("s_cmp_ge_u32 s97, %[ht]")
    e.emit("s_cbranch_scc1 L_tail_%=")
    e.emit("L_loop_%=:")
    for s in range(NSTAGE):
        advance_k(e)
        half_step(e, s, dma=True, prefetch_next=True, vmcnt=8, barrier=True)
    e.forget_bound()                       # the loop head is reached from two places
    e.emit("s_add_u32 s97, s97, 4")
    e.emit("s_cmp_lt_u32 s97, %[ht]")
    e.emit("s_cbranch_scc1 L_loop_%=")
    e.emit("L_tail_%=:")
    e.forget_bound()
    advance_k(e)
    half_step(e, 0, dma=True, prefetch_next=True, vmcnt=8, barrier=True)      # fetches the last tile
    half_step(e, 1, dma=False, prefetch_next=True, vmcnt=0, barrier=True)
    half_step(e, 2, dma=False, prefetch_next=True, vmcnt=None, barrier=False)
    half_step(e, 3, dma=False, prefetch_next=False, vmcnt=None, barrier=False)
    print("// Generated by gen_gemm_asm.py -- do not edit.")
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
H_WA, H_XA, H_WB, H_XB = 64, 80, 88, 104
H_BASE, H_CUR = 112, 122
H_WVOFF, H_XVOFF = 116, 120
H_STAGE = 0x6000


def main_half():
    e = Emitter()
    e.emit("; ======== setup ========")
    e.emit("v_mov_b32 v%d, %%[wb]" % (H_BASE + 0))
    e.emit("v_xor_b32 v%d, 0x20, %%[wb]" % (H_BASE + 1))
    e.emit("v_mov_b32 v%d, %%[xb]" % (H_BASE + 2))
    e.emit("v_xor_b32 v%d, 0x20, %%[xb]" % (H_BASE + 3))
    e.emit("v_mov_b32 v%d, %%[wv0]" % H_WVOFF)
    e.emit("v_mov_b32 v%d, %%[xv0]" % H_XVOFF)
    for i in range(1, 4):
        e.emit("v_add_u32 v%d, %%[w64], v%d" % (H_WVOFF + i, H_WVOFF + i - 1))
    e.emit("v_add_u32 v%d, %%[x64], v%d" % (H_XVOFF + 1, H_XVOFF))
    for r in range(4):
        e.emit("v_mov_b32 v%d, 0" % (H_WA + r))
    e.emit("s_nop 7")      # VALU result -> MFMA source operand
    for i in range(4):
        for j in range(2):
            e.emit("v_mfma_f32_32x32x16_bf16 %%[c%d%d], %s, %s, 0" % (i, j, vreg4(H_WA), vreg4(H_WA)))
    e.emit("s_mov_b32 s94, %[m0b]")
    e.emit("s_mov_b32 s92, 0")
    e.emit("s_mov_b32 s93, 0")
    e.emit("s_mov_b32 s96, 0")
    e.emit("s_mov_b32 s98, 0")

    def dma(k):
        """k-th of the wave's six loads of the tile at stage offset s93: (M0 update, load)."""
        m0 = "s_add_u32 m0, s94, s93" if k == 0 else "s_add_u32 m0, m0, 0x1000"
        if k < 4:
            ld = "buffer_load_dwordx4 v%d, %%[wres], s96 offen lds" % (H_WVOFF + k)
        else:
            ld = "buffer_load_dwordx4 v%d, %%[xres], s98 offen lds" % (H_XVOFF + k - 4)
        return m0, ld

    def rotate(reg):
        e.emit("s_add_u32 s%d, s%d, 0x%x" % (reg, reg, H_STAGE))
        e.emit("s_cmp_eq_u32 s%d, 0x%x" % (reg, 3 * H_STAGE))
        e.emit("s_cselect_b32 s%d, 0, s%d" % (reg, reg))

    e.emit("; ======== prologue: tiles 0, 1 -> stages 0, 1 ========")
    def advance_k_clamped():
        # The loads run two tiles ahead of the multiply, so the last two half-steps ask for tiles
        # past the end of K: they fetch the last tile again (the range check of a buffer
        # descriptor does not cover the scalar offset, so the offset itself has to stay inside).
        advance_k(e)
        e.emit("s_min_u32 s96, s96, %[wkmax]")
        e.emit("s_min_u32 s98, s98, %[xkmax]")

    for t in range(2):
        for k in range(6):
            m0, ld = dma(k)
            e.emit(m0)
            e.emit("s_nop 0")
            e.emit(ld)
        rotate(93)
        advance_k_clamped()
    e.emit("s_waitcnt vmcnt(6)")           # tile 0 has landed
    e.emit("s_barrier")

    def reads(kk, wset, xset):
        out = [(wset + 4 * b, H_CUR + kk, b * 2048) for b in range(4)]
        out += [(xset + 4 * b, H_CUR + 2 + kk, 0x4000 + b * 2048) for b in range(2)]
        # first the pair the first MFMA needs
        return [out[0], out[4], out[5], out[1], out[2], out[3]]

    def cur_addresses():
        for r in range(4):
            e.emit("v_add_u32 v%d, s92, v%d" % (H_CUR + r, H_BASE + r))

    def mfmas(wset, xset, tracked, pending, dma_from):
        """Eight MFMAs on one fragment set; `pending` LDS reads and the DMA loads
        dma_from, dma_from + 1, dma_from + 2 go behind them."""
        n_dma = 0
        m = 0
        for i in range(4):
            for j in range(2):
                if tracked:
                    e.need(wset + 4 * i, xset + 4 * j)
                d = dma_from + n_dma if (dma_from is not None and m % 2 == 0 and n_dma < 3) else None
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
        # vmcnt(6): everything but the loads just issued, i.e. the next tile, has landed.
        # lgkmcnt(0): my reads of this tile are done before anybody may overwrite its stage.
        e.emit("s_waitcnt vmcnt(6) lgkmcnt(0)")
        e.emit("s_barrier")

    # The pipeline is skewed by one k-phase: a half-step starts by reading its tile's k-phase-0
    # fragments (set A) and multiplies the PREVIOUS tile's k-phase 1 (set B, read a half-step
    # ago) while they arrive; then k-phase 0 on set A while k-phase 1 is read into set B.
    e.emit("; ======== half-step 0: no previous tile ========")
    cur_addresses()
    for r in reads(0, H_WA, H_XA):
        e.read(*r)
    mfmas(H_WA, H_XA, True, reads(1, H_WB, H_XB), 0)
    # the three remaining loads of tile 2 without MFMAs to hide behind
    for k in range(3, 6):
        e.emit(dma(k)[0])
        e.emit("s_nop 0")
        e.emit(dma(k)[1])
    end_of_half_step()
    e.emit("s_mov_b32 s97, 1")
    e.emit("s_cmp_ge_u32 s97, %[ht]")
    e.emit("s_cbranch_scc1 L_last_%=")
    e.emit("L_loop_%=:")
    cur_addresses()
    for r in reads(0, H_WA, H_XA):
        e.read(*r)
    e.emit("s_waitcnt lgkmcnt(6)")         # set B (read during the previous half-step) is complete
    e.forget_bound()
    e.guaranteed = 6
    mfmas(H_WB, H_XB, False, [], 0)
    mfmas(H_WA, H_XA, True, reads(1, H_WB, H_XB), 3)
    end_of_half_step()
    e.emit("s_add_u32 s97, s97, 1")
    e.emit("s_cmp_lt_u32 s97, %[ht]")
    e.emit("s_cbranch_scc1 L_loop_%=")
    e.emit("L_last_%=:")
    e.emit("s_waitcnt lgkmcnt(0)")
    e.emit("; ======== k-phase 1 of the last tile ========")
    mfmas(H_WB, H_XB, False, [], None)
    e.emit("s_waitcnt vmcnt(0)")
    e.emit("s_barrier")
    print("// Generated by gen_gemm_asm.py half -- do not edit.")
    for ln in e.lines:
        print('"%s\\n"' % ln)


if __name__ == "__main__":
    import sys
    if len(sys.argv) > 1 and sys.argv[1] == "half":
        main_half()
    else:
        main()
