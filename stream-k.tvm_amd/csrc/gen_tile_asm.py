#!/usr/bin/env python3
"""Writes tile_f16_asm_gen.h: the K loop of the four-wave 256 x 256 x 64 tile kernel as one block of gfx950
assembly (used by tile_f16_asm.h inside an `asm volatile` statement).

    python3 gen_tile_asm.py > tile_f16_asm_gen.h        (the Makefile does this when the script changes)

Why assembly: each of the four waves owns a 128 x 128 block of C, 256 fp32 accumulators per lane, which must
live in the accumulation registers a[0:255] for the whole loop while the 256 architectural registers hold
operand fragments.  The compiler will not keep that assignment (it moves accumulators between the two files
inside the loop), so the loop is written out with fixed registers:

  a[(8 i + j) 4 .. +3]   16 x 16 block (i, j) of the wave's 128 x 128 result (i: rows of A, j: rows of B)
  v[128:159] v[160:191]  A / B fragments of K-step 0 (eight 16-row blocks each, four registers per block)
  v[192:223] v[224:255]  A / B fragments of K-step 1
  v[120:121]             per-lane byte offsets of the A / B loads of this iteration
  s[80:87]               loop state (see the text)

One iteration (stage `cur` of the two 64 KB LDS stages holds its tiles, `nxt` the next iteration's):
  block 0   64 MFMAs on the K-step-0 fragments; the 16 fragment reads of K-step 1 (from cur) ride along
  sync      wait for them, wait for this wave's direct-to-LDS loads into nxt, barrier
  block 1   64 MFMAs on the K-step-1 fragments; along ride the 16 loads of iteration it + 2 into cur (which
            every wave has finished reading) and the 16 fragment reads of K-step 0 of nxt
The loads of iterations past the segment get an out-of-range offset (they fetch nothing and zero a stage
nobody reads), so the loop has no branch but its own back edge.

NN layout (B is [K, N] row-major; SK_TILE_ASM_LOOP_NN): the B half of a stage is 64 K-rows of 512 bytes, a
wave-wide load fills two of them (row group g = wave + 4 x: K-rows 2 g, 2 g + 1), 16-byte chunk c of K-row k sits
at position c ^ (4 (k & 3)) ^ (2 ((k >> 3) & 1)).  Bit 3 of a lane's K-row is the parity of x, so the lane fetches
one of two global chunks: v121 for even x, v122 for odd x.  A 16-column block of B is read with two transposing
8-byte reads per K-step (K-rows 8 g' .. + 3 and + 4 .. + 7 for lane group g'), from one address register per block
(%[rbt0] .. %[rbt7]; the swizzle makes the blocks' addresses differ by an XOR, not a sum): K-step 1 is 32 rows =
16384 bytes further.  Per iteration the global offset of B advances by %[kbs] = 64 rows.
"""

A0, B0, A1, B1 = 128, 160, 192, 224     # first registers of the fragment buffers
VOA, VOB, VOB1 = 120, 121, 122          # v120 / v121 (/ v122, NN: odd row groups of B): load offsets of this iteration
S_IT, S_KA, S_KB, S_T, S_OOB, S_M0, S_LDS, S_T2 = 80, 81, 82, 83, 84, 85, 86, 87


def emit(lines, text):
    lines.append(text)


def mfma(lines, i, j, a_base, b_base):
    c = (8 * i + j) * 4
    emit(lines, f'MF " a[{c}:{c + 3}], v[{b_base + 4 * j}:{b_base + 4 * j + 3}], v[{a_base + 4 * i}:{a_base + 4 * i + 3}], a[{c}:{c + 3}]')


NN = False   # set by main() while it writes the NN form of the loop


def frag_read(lines, f, a_base, b_base, addr_a, addr_b, kk=0):
    """fragment f: 0..7 blocks of A, 8.. blocks of B; 16 rows of 128 bytes per block.  NN: f = 8 + 2 g + h is
    half h of block g of B, four K-rows of K-step kk"""
    if f < 8:
        emit(lines, f'"ds_read_b128 v[{a_base + 4 * f}:{a_base + 4 * f + 3}], {addr_a} offset:{f * 2048}')
    elif not NN:
        g = f - 8
        emit(lines, f'"ds_read_b128 v[{b_base + 4 * g}:{b_base + 4 * g + 3}], {addr_b} offset:{g * 2048}')
    else:
        g, h = (f - 8) // 2, (f - 8) % 2
        r = b_base + 4 * g + 2 * h
        emit(lines, f'"ds_read_b64_tr_b16 v[{r}:{r + 1}], %[rbt{g}] offset:{kk * 16384 + h * 2048}')


def n_frags():
    return 24 if NN else 16


def dma(lines, x, first):
    """load x of a stage: 0..7 row groups of A, 8..15 of B (a wave's groups are 4 KB apart in LDS);
    s[S_T] walks the global offsets of the groups, s[S_LDS] is the stage's LDS address for this wave"""
    if x == 0:
        emit(lines, f'"s_mov_b32 s{S_T}, s{S_KA}')
    if x == 8:
        emit(lines, f'"s_mov_b32 s{S_T}, s{S_KB}')
    lds_off = (x * 4096) if x < 8 else (32768 + (x - 8) * 4096)
    emit(lines, f'"s_add_u32 m0, s{S_LDS}, {lds_off}')
    emit(lines, '"s_nop 0')
    if x < 8:
        emit(lines, f'"buffer_load_dwordx4 v{VOA}, %[rsa], s{S_T} offen lds')
        emit(lines, f'"s_add_u32 s{S_T}, s{S_T}, %[gas]')
    else:
        vob = VOB1 if (NN and x % 2 == 1) else VOB
        emit(lines, f'"buffer_load_dwordx4 v{vob}, %[rsb], s{S_T} offen lds')
        emit(lines, f'"s_add_u32 s{S_T}, s{S_T}, %[gbs]')


def offsets_for(lines, ahead):
    """v120 / v121 = the lane offsets, pushed out of range if iteration it + ahead is past the segment"""
    emit(lines, f'"s_add_u32 s{S_T2}, s{S_IT}, {ahead}')
    emit(lines, f'"s_cmp_lt_u32 s{S_T2}, %[n]')
    emit(lines, f'"s_cselect_b32 s{S_OOB}, 0, 0x80000000')
    emit(lines, f'"v_or_b32 v{VOA}, s{S_OOB}, %[voa]')
    emit(lines, f'"v_or_b32 v{VOB}, s{S_OOB}, %[vob]')
    if NN:
        emit(lines, f'"v_or_b32 v{VOB1}, s{S_OOB}, %[vob1]')


def mfma_order():
    # walk the 8 x 8 blocks so that consecutive instructions share one operand
    order = []
    for i in range(8):
        js = range(8) if i % 2 == 0 else range(7, -1, -1)
        order += [(i, j) for j in js]
    return order


def slots(count, total, first, every):
    """MFMA indices after which `count` riders are issued: every `every`-th instruction from `first` on"""
    out = [first + k * every for k in range(count)]
    assert out[-1] < total, (count, total, first, every)
    return out


def loop_text(nn):
    """the lines of the loop for the NT (nn = False) or the NN layout"""
    global NN
    NN = nn
    import os
    # where the fragment reads and the loads ride along the 64 MFMAs of a block (tunables of the schedule)
    # (measured at 8192^3 on random operands, each against the eight-wave kernel in the same run: the defaults
    # 1.07-1.08 x; all 16 loads in the first 16 or 32 MFMA slots behind the barrier 0.98 x -- the wave then stalls
    # at the texture addresser, and with one wave per SIMD that is a stalled matrix pipe; loads every third slot
    # 1.05 x; later or denser fragment reads, a partial wait at the loop top, MFMAs issued ahead of the barrier:
    # within 1 % of the defaults.  The same loop on four 32 KB buffers with a barrier per K-step of 32: 1.00 x.)
    # NN: 8 + 16 reads per K-step, on the even slots; the loads keep the odd slots 3, 7, ...
    nf = n_frags()
    if nn:
        rd0 = slots(nf, 64, 0, 2)
        rd1 = slots(nf, 64, 0, 2)
    else:
        rd0 = slots(nf, 64, int(os.environ.get("SK_ASM_RD0_FIRST", 0)), int(os.environ.get("SK_ASM_RD0_EVERY", 3)))
        rd1 = slots(nf, 64, int(os.environ.get("SK_ASM_RD1_FIRST", 1)), int(os.environ.get("SK_ASM_RD1_EVERY", 4)))
    ld1 = slots(16, 64, int(os.environ.get("SK_ASM_LD1_FIRST", 3)), int(os.environ.get("SK_ASM_LD1_EVERY", 4)))
    kb_step = "%[kbs]" if nn else "128"
    frag_addrs = ["%[ra0]", "%[ra1]"] + ([f"%[rbt{g}]" for g in range(8)] if nn else ["%[rb0]", "%[rb1]"])
    L = []
    # ---- accumulators start at zero
    for r in range(256):
        emit(L, f'"v_accvgpr_write_b32 a{r}, 0')
    # ---- prologue: both stages requested, wait for the first
    emit(L, f'"s_mov_b32 s{S_IT}, 0')
    emit(L, f'"s_mov_b32 s{S_LDS}, %[lds]')
    emit(L, f'"s_mov_b32 s{S_KA}, %[ga0]')
    emit(L, f'"s_mov_b32 s{S_KB}, %[gb0]')
    offsets_for(L, 0)
    for x in range(16):
        dma(L, x, True)
    emit(L, f'"s_add_u32 s{S_KA}, s{S_KA}, 128')
    emit(L, f'"s_add_u32 s{S_KB}, s{S_KB}, {kb_step}')
    emit(L, f'"s_xor_b32 s{S_LDS}, s{S_LDS}, 0x10000')
    offsets_for(L, 1)
    for x in range(16):
        dma(L, x, False)
    emit(L, f'"s_add_u32 s{S_KA}, s{S_KA}, 128')
    emit(L, f'"s_add_u32 s{S_KB}, s{S_KB}, {kb_step}')
    emit(L, f'"s_xor_b32 s{S_LDS}, s{S_LDS}, 0x10000')
    emit(L, '"s_waitcnt vmcnt(16)')
    emit(L, '"s_barrier')
    for f in range(nf):
        frag_read(L, f, A0, B0, "%[ra0]", "%[rb0]", 0)
    emit(L, '"s_nop 7')   # accumulator writes above are long done; cheap insurance before the first MFMA
    # ---- the loop
    emit(L, '"L_sk_loop%=:')
    # the K-step-0 fragments were requested in the order A0..A7, B0..B7: the first MFMAs need A0 and the first
    # B blocks only, the youngest reads (the last B blocks) get until MFMA `late_at` to arrive
    late = int(os.environ.get("SK_ASM_TOP_LATE", 0))
    late_at = int(os.environ.get("SK_ASM_TOP_LATE_AT", 4))
    emit(L, f'"s_waitcnt lgkmcnt({late})')
    order = mfma_order()
    for m, (i, j) in enumerate(order):
        if late and m == late_at:
            emit(L, '"s_waitcnt lgkmcnt(0)')
        mfma(L, i, j, A0, B0)
        if m in rd0:
            frag_read(L, rd0.index(m), A1, B1, "%[ra1]", "%[rb1]", 1)
    emit(L, '"s_waitcnt lgkmcnt(0)')
    # the first MFMAs of block 1 need the K-step-1 fragments only: issued ahead of the barrier they keep the
    # matrix pipe busy while the wave waits there
    early = int(os.environ.get("SK_ASM_EARLY", 0))
    for m in range(early):
        mfma(L, *order[m], A1, B1)
    emit(L, '"s_waitcnt vmcnt(0)')
    emit(L, '"s_barrier')
    offsets_for(L, 2)
    # from here on the fragment addresses point at the other stage
    for reg in frag_addrs:
        emit(L, f'"v_xor_b32 {reg}, 0x10000, {reg}')
    for m, (i, j) in enumerate(order):
        if m >= early:
            mfma(L, i, j, A1, B1)
        if m in ld1:
            dma(L, ld1.index(m), False)
        if m in rd1:
            frag_read(L, rd1.index(m), A0, B0, "%[ra0]", "%[rb0]", 0)
    emit(L, f'"s_add_u32 s{S_KA}, s{S_KA}, 128')
    emit(L, f'"s_add_u32 s{S_KB}, s{S_KB}, {kb_step}')
    emit(L, f'"s_xor_b32 s{S_LDS}, s{S_LDS}, 0x10000')
    emit(L, f'"s_add_u32 s{S_IT}, s{S_IT}, 1')
    emit(L, f'"s_cmp_lt_u32 s{S_IT}, %[n]')
    emit(L, '"s_cbranch_scc1 L_sk_loop%=')
    # ---- drain: the empty loads of the last two iterations still write LDS; the accumulators must have left
    # the matrix pipe before ordinary instructions read them
    emit(L, '"s_waitcnt vmcnt(0) lgkmcnt(0)')
    for _ in range(3):
        emit(L, '"s_nop 7')
    return L


class LdsTracker:
    """issue order of the fragment reads and the s_waitcnt lgkmcnt(n) a consumer needs (reads return in order)"""

    def __init__(self, outstanding):
        self.q = list(outstanding)      # tags still possibly in flight, oldest first

    def issue(self, tag):
        self.q.append(tag)

    def need(self, lines, tags):
        last = max((k for k, t in enumerate(self.q) if t in tags), default=-1)
        if last < 0:
            return
        allowed = len(self.q) - 1 - last
        emit(lines, f'"s_waitcnt lgkmcnt({min(allowed, 15)})')
        self.q = self.q[last + 1:] if allowed <= 15 else self.q[len(self.q) - 15:]

    def drain(self, lines):
        emit(lines, '"s_waitcnt lgkmcnt(0)')
        self.q = []


def loop_text_f8():
    """fp8 operands (SK_TILE_ASM_LOOP_F8): one v_mfma_f32_16x16x128_f8f6f4 per accumulator block and iteration, on
    32-byte fragments made of the two 16-byte fragments of the 16-bit loop (which K-values a lane's bytes stand for
    does not matter as long as A and B agree).  Block i of A lives in v[128 + 8 i .. + 7], block j of B in
    v[192 + 8 j .. + 7]: all 128 fragment registers hold one iteration, so there is no second set to read ahead
    into.  Instead an iteration runs in two phases of 32 MFMAs (32 cycles each):
      phase 1   blocks i = 0..3 of A against j = 7..0; the fragments of i = 4..7 (same stage) ride along
      sync      wait for them and for this wave's loads into the other stage, barrier
      phase 2   blocks i = 4..7 against j = 7..0; along ride the 16 loads of iteration it + 2 into the stage just
                read, the next iteration's fragments of i = 0..3, and its fragment of B block j once the four
                MFMAs that use the old one have been issued and a further one behind them
    The waits before the MFMAs are computed from the order in which the reads were issued."""
    global NN
    NN = False
    A8 = lambda i: 128 + 8 * i
    B8 = lambda j: 192 + 8 * j
    L = []

    def read_half(tr, which, blk, h, stage_next):
        base = (A8 if which == "A" else B8)(blk) + 4 * h
        addr = ("%[ra1]" if h else "%[ra0]") if which == "A" else ("%[rb1]" if h else "%[rb0]")
        emit(L, f'"ds_read_b128 v[{base}:{base + 3}], {addr} offset:{blk * 2048}')
        tr.issue((which, blk))

    def mf(i, j):
        c = (8 * i + j) * 4
        emit(L, f'MF " a[{c}:{c + 3}], v[{B8(j)}:{B8(j) + 7}], v[{A8(i)}:{A8(i) + 7}], a[{c}:{c + 3}] " MOD "')

    for r in range(256):
        emit(L, f'"v_accvgpr_write_b32 a{r}, 0')
    emit(L, f'"s_mov_b32 s{S_IT}, 0')
    emit(L, f'"s_mov_b32 s{S_LDS}, %[lds]')
    emit(L, f'"s_mov_b32 s{S_KA}, %[ga0]')
    emit(L, f'"s_mov_b32 s{S_KB}, %[gb0]')
    for ahead in (0, 1):
        offsets_for(L, ahead)
        for x in range(16):
            dma(L, x, ahead == 0)
        emit(L, f'"s_add_u32 s{S_KA}, s{S_KA}, 128')
        emit(L, f'"s_add_u32 s{S_KB}, s{S_KB}, 128')
        emit(L, f'"s_xor_b32 s{S_LDS}, s{S_LDS}, 0x10000')
    emit(L, '"s_waitcnt vmcnt(16)')
    emit(L, '"s_barrier')
    tr = LdsTracker([])
    for i in range(4):
        for h in range(2):
            read_half(tr, "A", i, h, False)
    for j in range(7, -1, -1):
        for h in range(2):
            read_half(tr, "B", j, h, False)
    emit(L, '"s_nop 7')
    emit(L, '"L_sk_loop%=:')
    # both ways into the loop end with the four reads of B blocks 1 and 0
    emit(L, '"s_waitcnt lgkmcnt(4)')
    tr = LdsTracker([("B", 1), ("B", 1), ("B", 0), ("B", 0)])
    # ---- phase 1
    pending = [("A", i, h) for i in range(4, 8) for h in range(2)]
    m = 0
    for j in range(7, -1, -1):
        for i in range(4):
            tr.need(L, {("A", i), ("B", j)})
            mf(i, j)
            if m % 2 == 0 and pending:
                w, blk, h = pending.pop(0)
                read_half(tr, w, blk, h, False)
            m += 1
    assert not pending
    tr.drain(L)
    emit(L, '"s_waitcnt vmcnt(0)')
    emit(L, '"s_barrier')
    offsets_for(L, 2)
    for reg in ("%[ra0]", "%[ra1]", "%[rb0]", "%[rb1]"):
        emit(L, f'"v_xor_b32 {reg}, 0x10000, {reg}')
    # ---- phase 2
    a_next = [("A", i, h) for i in range(4) for h in range(2)]
    b_next = {}      # slot -> reads of the next iteration's B fragments
    for j in range(7, -1, -1):
        s0 = 4 * (7 - j) + 5
        b_next.setdefault(s0, []).append(("B", j, 0))
        b_next.setdefault(s0 + 1, []).append(("B", j, 1))
    m = 0
    for j in range(7, -1, -1):
        for i in range(4, 8):
            tr.need(L, {("A", i), ("B", j)})
            mf(i, j)
            if m % 2 == 1:
                dma(L, m // 2, False)
            if m % 2 == 0 and a_next:
                w, blk, h = a_next.pop(0)
                read_half(tr, w, blk, h, True)
            for (w, blk, h) in b_next.pop(m, []):
                read_half(tr, w, blk, h, True)
            m += 1
    for slot in sorted(b_next):
        for (w, blk, h) in b_next[slot]:
            read_half(tr, w, blk, h, True)
    assert not a_next and tr.q[-4:] == [("B", 1), ("B", 1), ("B", 0), ("B", 0)]
    emit(L, f'"s_add_u32 s{S_KA}, s{S_KA}, 128')
    emit(L, f'"s_add_u32 s{S_KB}, s{S_KB}, 128')
    emit(L, f'"s_xor_b32 s{S_LDS}, s{S_LDS}, 0x10000')
    emit(L, f'"s_add_u32 s{S_IT}, s{S_IT}, 1')
    emit(L, f'"s_cmp_lt_u32 s{S_IT}, %[n]')
    emit(L, '"s_cbranch_scc1 L_sk_loop%=')
    emit(L, '"s_waitcnt vmcnt(0) lgkmcnt(0)')
    for _ in range(3):
        emit(L, '"s_nop 7')
    return L


def main():
    print("// Generated by gen_tile_asm.py -- do not edit; see that file for the register plan and the schedule.")
    print("// SK_TILE_ASM_LOOP(MF) / SK_TILE_ASM_LOOP_NN(MF): the loop text for the NT / NN layout, MF = the MFMA")
    print("// mnemonic as a string literal.")
    print("#pragma once")
    for name, nn in (("SK_TILE_ASM_LOOP", False), ("SK_TILE_ASM_LOOP_NN", True)):
        print(f"#define {name}(MF) \\")
        for text in loop_text(nn):
            print(f"  {text}\\n\\t\" \\")
        print("  \"\"")
    print("// SK_TILE_ASM_LOOP_F8(MF, MOD): fp8 operands; MOD = the format modifiers of the MFMA (\"\" for e4m3)")
    print("#define SK_TILE_ASM_LOOP_F8(MF, MOD) \\")
    for text in loop_text_f8():
        print(f"  {text}\\n\\t\" \\")
    print("  \"\"")
    clob = [f'"a{r}"' for r in range(256)] + [f'"v{r}"' for r in range(120, 256)] + [f'"s{r}"' for r in range(80, 88)]
    print("#define SK_TILE_ASM_CLOBBERS \\")
    for k in range(0, len(clob), 16):
        tail = ", \\" if k + 16 < len(clob) else ""
        print("  " + ", ".join(clob[k:k + 16]) + tail)


if __name__ == "__main__":
    main()
