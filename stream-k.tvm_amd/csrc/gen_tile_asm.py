#!/usr/bin/env python3
"""Writes tile_f16_asm_gen.h: the assembly text of the four-wave 256 x 256 x 64 tile kernel (tile_f16_asm.h uses
each macro inside an `asm volatile` statement).

    python3 gen_tile_asm.py > tile_f16_asm_gen.h        (the Makefile does this when the script changes)

Why assembly: each of the four waves owns a 128 x 128 block of C, 256 fp32 accumulators per lane, which must
live in the accumulation registers a[0:255] for the whole loop while the 256 architectural registers hold
operand fragments.  The compiler will not keep that assignment (it moves accumulators between the two files
inside the loop), so the loop is written out with fixed registers:

  a[(8 i + j) 4 .. +3]   16 x 16 block (i, j) of the wave's 128 x 128 result (i: rows of A, j: rows of B)
  v[128:159] v[160:191]  A / B fragments of K-step 0 (eight 16-row blocks each, four registers per block)
  v[192:223] v[224:255]  A / B fragments of K-step 1
  v[120:122]             per-lane byte offsets of the A / B loads of this iteration
  s[80:87]               loop state (see the text)

Three pieces of text per layout:

  SK_TILE_ASM_LOADS*   the 16 direct-to-LDS loads of one 64 KB stage (8 row groups of A, 8 of B per wave).  A segment
                       starts with the loads of its first two stages; the first stage of the NEXT segment is requested
                       before the epilogue of the current one, so that its latency hides behind the stores of C.
  SK_TILE_ASM_LOOP*    zero the accumulators, wait for the first stage, run the K loop, drain.
  SK_TILE_ASM_STORE*   the epilogue of a tile that needs no edge handling: accumulators -> 16-bit pairs -> a small
                       per-wave patch of LDS behind the stages -> 16-byte stores of whole row pieces.  The stages are
                       not touched, which is what allows the next segment's loads to be in flight.

One iteration of the loop (stage `cur` of the two LDS stages holds its tiles, `nxt` the next iteration's):
  block 0   64 MFMAs on the K-step-0 fragments.  Riding along: the last six A fragments of K-step 0 (read at the top,
            each needed eight MFMAs after the previous one), the 16 fragment reads of K-step 1, the lane offsets of
            the loads to come, one of the two stage flips of the fragment addresses
  sync      wait for those reads and for this wave's loads into nxt, barrier
  block 1   64 MFMAs on the K-step-1 fragments.  Riding along: the 16 loads of iteration it + 2 into cur (which
            every wave has finished reading), the first ten fragment reads of K-step 0 of nxt, the other flips
Riders are dealt out ONE GROUP PER MFMA GAP (a gap is the 16 cycles an MFMA occupies the matrix pipe; the wave issues
about one other instruction per four cycles in it).  Counters: with the four instructions of a load in one gap, as an
earlier version had them, every load cost ~10 cycles of matrix-pipe time, and the scalar work bunched at the barrier
and at the loop end another ~90 cycles per iteration; an MFMA that waits for a fragment waits only for the reads it
needs (the waits are computed from the issue order: LDS reads return in order).
The loads of iterations past the segment get an out-of-range offset (they fetch nothing and zero a stage nobody
reads), so the loop has no branch but its own back edge.

NN layout (B is [K, N] row-major; SK_TILE_ASM_*_NN): the B half of a stage is 64 K-rows of 512 bytes, a
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

ROLL = 6    # A fragments of K-step 0 that are read at the top of their own block 0 instead of in the block before
# (measured at 8192^3, cycles per CU from SQ_BUSY_CU_CYCLES: three gaps per load -- m0, load, offset advance -- against
# two with the scalar pair sharing a gap: within 0.2 %; the NN loop has 24 fragment reads per K-step and takes two)
RD0_FIRST, RD0_LAST = 8, 50   # gaps of block 0 over which the K-step-1 fragment reads are spread


def mfma_order():
    # walk the 8 x 8 blocks so that consecutive instructions share one operand
    order = []
    for i in range(8):
        js = range(8) if i % 2 == 0 else range(7, -1, -1)
        order += [(i, j) for j in js]
    return order


class LdsTracker:
    """issue order of the fragment reads and the s_waitcnt lgkmcnt(n) a consumer needs (reads return in order)"""

    def __init__(self, outstanding=()):
        self.q = list(outstanding)      # tags still possibly in flight, oldest first

    def issue(self, tag):
        self.q.append(tag)

    def wait_for(self, tags):
        """text of the wait an instruction that consumes `tags` needs, or None"""
        last = max((k for k, t in enumerate(self.q) if t in tags), default=-1)
        if last < 0:
            return None
        allowed = len(self.q) - 1 - last
        self.q = self.q[last + 1:] if allowed <= 15 else self.q[len(self.q) - 15:]
        return f'"s_waitcnt lgkmcnt({min(allowed, 15)})'


def load_parts(x, nn, voa, vob, vob1, lds, ka, kb):
    """load x of a stage: 0..7 row groups of A, 8..15 of B (a wave's groups are 4 KB apart in LDS).  Returns
    (instructions that go before the m0 write, the m0 write, the load, the advance of the global offset);
    s[S_T] walks the global offsets of the groups, `lds` is the stage's LDS address for this wave"""
    pre = []
    if x == 0:
        pre.append(f'"s_mov_b32 s{S_T}, {ka}')
    if x == 8:
        pre.append(f'"s_mov_b32 s{S_T}, {kb}')
    lds_off = (x * 4096) if x < 8 else (32768 + (x - 8) * 4096)
    m0 = f'"s_add_u32 m0, {lds}, {lds_off}'
    if x < 8:
        ld = f'"buffer_load_dwordx4 {voa}, %[rsa], s{S_T} offen lds'
        adv = f'"s_add_u32 s{S_T}, s{S_T}, %[gas]'
    else:
        ld = f'"buffer_load_dwordx4 {vob1 if (nn and x % 2 == 1) else vob}, %[rsb], s{S_T} offen lds'
        adv = f'"s_add_u32 s{S_T}, s{S_T}, %[gbs]'
    return pre, m0, ld, adv


def stage_loads_text(nn):
    """the 16 loads of one stage, back to back (operands: the stage's LDS address, global offsets and lane offsets)"""
    L = []
    for x in range(16):
        pre, m0, ld, adv = load_parts(x, nn, "%[voa]", "%[vob]", "%[vob1]", "%[lds]", "%[ga]", "%[gb]")
        L += pre + [m0, '"s_nop 0', ld]
        if x not in (7, 15):
            L.append(adv)
    return L


def offsets_for(nn, ahead):
    """v120 / v121 = the lane offsets, pushed out of range if iteration it + ahead is past the segment"""
    out = [f'"s_add_u32 s{S_T2}, s{S_IT}, {ahead}', f'"s_cmp_lt_u32 s{S_T2}, %[n]', f'"s_cselect_b32 s{S_OOB}, 0, 0x80000000',
           f'"v_or_b32 v{VOA}, s{S_OOB}, %[voa]', f'"v_or_b32 v{VOB}, s{S_OOB}, %[vob]']
    if nn:
        out.append(f'"v_or_b32 v{VOB1}, s{S_OOB}, %[vob1]')
    return out


def loop_entry(L, nn):
    """accumulators to zero while the first stage is on its way; the loop's state; wait for that stage"""
    for r in range(256):
        L.append(f'"v_accvgpr_write_b32 a{r}, 0')
    L.append(f'"s_mov_b32 s{S_IT}, 0')
    L.append(f'"s_mov_b32 s{S_LDS}, %[lds]')
    # the loads in the loop start with iteration 2
    L.append(f'"s_add_u32 s{S_KA}, %[ga0], 256')
    if nn:
        L.append(f'"s_lshl_b32 s{S_T2}, %[kbs], 1')
        L.append(f'"s_add_u32 s{S_KB}, %[gb0], s{S_T2}')
    else:
        L.append(f'"s_add_u32 s{S_KB}, %[gb0], 256')
    L.append('"s_waitcnt vmcnt(16)')     # (the 16 youngest vector memory operations are the loads of the second stage)
    L.append('"s_barrier')


def loop_text(nn):
    """the lines of the loop for the NT (nn = False) or the NN layout"""
    L = []
    e = L.append
    kb_step = "%[kbs]" if nn else "128"
    order = mfma_order()

    def mf(i, j, ab, bb):
        c = (8 * i + j) * 4
        return f'MF " a[{c}:{c + 3}], v[{bb + 4 * j}:{bb + 4 * j + 3}], v[{ab + 4 * i}:{ab + 4 * i + 3}], a[{c}:{c + 3}]'

    # fragment reads as (tag, text); 16 rows of 128 bytes per block of A (NT: of B too)
    def read_a(i, kk):
        ab, addr = (A0, "%[ra0]") if kk == 0 else (A1, "%[ra1]")
        return (("A", kk, i), f'"ds_read_b128 v[{ab + 4 * i}:{ab + 4 * i + 3}], {addr} offset:{i * 2048}')

    def read_b(j, kk):
        bb = B0 if kk == 0 else B1
        if not nn:
            addr = "%[rb0]" if kk == 0 else "%[rb1]"
            return [(("B", kk, j), f'"ds_read_b128 v[{bb + 4 * j}:{bb + 4 * j + 3}], {addr} offset:{j * 2048}')]
        # NN: two halves of four K-rows each
        return [(("B", kk, j), f'"ds_read_b64_tr_b16 v[{bb + 4 * j + 2 * h}:{bb + 4 * j + 2 * h + 1}], %[rbt{j}] offset:{kk * 16384 + h * 2048}')
                for h in range(2)]

    def reads_in_need_order(kk):
        """A_0, B_0 .. B_7 (the first eight MFMAs need them in this order), then A_1 .. A_7 (one per eight MFMAs)"""
        seq = [read_a(0, kk)]
        for j in range(8):
            seq += read_b(j, kk)
        return seq + [read_a(i, kk) for i in range(1, 8)]

    loop_entry(L, nn)
    # the K-step-0 reads that block 1 of an iteration issues for the next one
    k0_reads = reads_in_need_order(0)
    n_ahead = len(k0_reads) - ROLL
    tr = LdsTracker()
    for tag, text in k0_reads[:n_ahead]:
        e(text)
        tr.issue(tag)
    at_top = list(tr.q)
    e('"s_nop 7')   # accumulator writes above are long done; cheap insurance before the first MFMA
    e('"L_sk_loop%=:')

    # ---- block 0
    tr = LdsTracker(at_top)
    plan = {}       # gap -> [(tag or None, [texts])]
    g = 0
    for tag, text in k0_reads[n_ahead:]:
        plan.setdefault(g, []).append((tag, [text]))
        g += 1
    k1_reads = reads_in_need_order(1)
    first = max(RD0_FIRST, g)
    for k, (tag, text) in enumerate(k1_reads):
        plan.setdefault(first + (k * (RD0_LAST - first)) // (len(k1_reads) - 1), []).append((tag, [text]))
    off = offsets_for(nn, 2)
    misc = [['"v_xor_b32 %[ra0], 0x10000, %[ra0]']]             # (behind the reads at the top, which use it)
    if not nn:
        misc.append(['"v_xor_b32 %[rb0], 0x10000, %[rb0]'])
    misc += [off[0:1], off[1:3]] + [[t] for t in off[3:]]        # (compare and select share a gap: nothing between them writes scc)
    free = [x for x in range(g, 62) if x not in plan]
    assert len(free) >= len(misc), (len(free), len(misc))
    for k, texts in enumerate(misc):
        plan.setdefault(free[(k * len(free)) // len(misc)], []).append((None, texts))
    for m, (i, j) in enumerate(order):
        w = tr.wait_for({("A", 0, i), ("B", 0, j)})
        if w:
            e(w)
        e(mf(i, j, A0, B0))
        for tag, texts in plan.get(m, []):
            L.extend(texts)
            if tag:
                tr.issue(tag)
    e('"s_waitcnt vmcnt(0) lgkmcnt(0)')
    e('"s_barrier')
    if nn:
        # one address register per block of B serves both K-steps: they flip between the reads of block 0 and block 1
        for j in range(8):
            e(f'"v_xor_b32 %[rbt{j}], 0x10000, %[rbt{j}]')

    # ---- block 1
    tr = LdsTracker()
    items = []      # (position in [0, 1), tie-break, tag or None, [texts])
    groups = []
    for x in range(16):
        pre, m0, ld, adv = load_parts(x, nn, f"v{VOA}", f"v{VOB}", f"v{VOB1}", f"s{S_LDS}", f"s{S_KA}", f"s{S_KB}")
        if nn:
            # two gaps per load: the advance behind load x - 1 shares the gap of the m0 write of load x
            groups += [([load_parts(x - 1, nn, "", "", "", "", "", "")[3]] if x not in (0, 8) else []) + pre + [m0], [ld]]
        else:
            groups += [pre + [m0], [ld]] + ([[adv]] if x not in (7, 15) else [])
    for k, texts in enumerate(groups):
        items.append(((k + 0.5) / len(groups), 0, None, texts))
    ahead = k0_reads[:n_ahead]
    for k, (tag, text) in enumerate(ahead):
        items.append((0.05 + 0.9 * (k + 0.5) / len(ahead), 1, tag, [text]))
    items.append((0.02, 2, None, ['"v_xor_b32 %[ra1], 0x10000, %[ra1]']))
    if not nn:
        items.append((0.5, 2, None, ['"v_xor_b32 %[rb1], 0x10000, %[rb1]']))
    items.sort(key=lambda t: (t[0], t[1]))
    tail = [[f'"s_add_u32 s{S_KA}, s{S_KA}, 128', f'"s_add_u32 s{S_KB}, s{S_KB}, {kb_step}'],
            [f'"s_xor_b32 s{S_LDS}, s{S_LDS}, 0x10000', f'"s_add_u32 s{S_IT}, s{S_IT}, 1'],
            [f'"s_cmp_lt_u32 s{S_IT}, %[n]', '"s_cbranch_scc1 L_sk_loop%=']]
    ngaps = 64 - len(tail)
    assert len(items) <= ngaps, (len(items), ngaps)
    plan = {}
    for k, it in enumerate(items):
        plan.setdefault((k * ngaps) // len(items), []).append((it[2], it[3]))
    for k, texts in enumerate(tail):
        plan.setdefault(ngaps + k, []).append((None, texts))
    for m, (i, j) in enumerate(order):
        w = tr.wait_for({("A", 1, i), ("B", 1, j)})
        if w:
            e(w)
        e(mf(i, j, A1, B1))
        for tag, texts in plan.get(m, []):
            L.extend(texts)
            if tag:
                tr.issue(tag)
    assert tr.q == at_top, (tr.q, at_top)            # both ways into the loop leave the same reads in flight
    for a, b in zip(L, L[1:]):                       # one instruction between an m0 write and the load that uses it
        assert not ("m0" in a and "buffer_load" in b), (a, b)
    # ---- drain: the empty loads of the last two iterations still write LDS; the accumulators must have left
    # the matrix pipe before ordinary instructions read them
    e('"s_waitcnt vmcnt(0) lgkmcnt(0)')
    for _ in range(3):
        e('"s_nop 7')
    return L


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
    A8 = lambda i: 128 + 8 * i
    B8 = lambda j: 192 + 8 * j
    L = []
    e = L.append

    def read_half(tr, which, blk, h):
        base = (A8 if which == "A" else B8)(blk) + 4 * h
        addr = ("%[ra1]" if h else "%[ra0]") if which == "A" else ("%[rb1]" if h else "%[rb0]")
        e(f'"ds_read_b128 v[{base}:{base + 3}], {addr} offset:{blk * 2048}')
        tr.issue((which, blk))

    def need(tr, tags):
        w = tr.wait_for(tags)
        if w:
            e(w)

    def mf(i, j):
        c = (8 * i + j) * 4
        e(f'MF " a[{c}:{c + 3}], v[{B8(j)}:{B8(j) + 7}], v[{A8(i)}:{A8(i) + 7}], a[{c}:{c + 3}] " MOD "')

    def dma(x):
        pre, m0, ld, adv = load_parts(x, False, f"v{VOA}", f"v{VOB}", f"v{VOB1}", f"s{S_LDS}", f"s{S_KA}", f"s{S_KB}")
        L.extend(pre + [m0, '"s_nop 0', ld, adv])

    loop_entry(L, False)
    tr = LdsTracker()
    for i in range(4):
        for h in range(2):
            read_half(tr, "A", i, h)
    for j in range(7, -1, -1):
        for h in range(2):
            read_half(tr, "B", j, h)
    e('"s_nop 7')
    e('"L_sk_loop%=:')
    # both ways into the loop end with the four reads of B blocks 1 and 0
    e('"s_waitcnt lgkmcnt(4)')
    tr = LdsTracker([("B", 1), ("B", 1), ("B", 0), ("B", 0)])
    # ---- phase 1
    pending = [("A", i, h) for i in range(4, 8) for h in range(2)]
    m = 0
    for j in range(7, -1, -1):
        for i in range(4):
            need(tr, {("A", i), ("B", j)})
            mf(i, j)
            if m % 2 == 0 and pending:
                w, blk, h = pending.pop(0)
                read_half(tr, w, blk, h)
            m += 1
    assert not pending
    e('"s_waitcnt vmcnt(0) lgkmcnt(0)')
    tr = LdsTracker()
    e('"s_barrier')
    L.extend(offsets_for(False, 2))
    for reg in ("%[ra0]", "%[ra1]", "%[rb0]", "%[rb1]"):
        e(f'"v_xor_b32 {reg}, 0x10000, {reg}')
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
            need(tr, {("A", i), ("B", j)})
            mf(i, j)
            if m % 2 == 1:
                dma(m // 2)
            if m % 2 == 0 and a_next:
                w, blk, h = a_next.pop(0)
                read_half(tr, w, blk, h)
            for (w, blk, h) in b_next.pop(m, []):
                read_half(tr, w, blk, h)
            m += 1
    for slot in sorted(b_next):
        for (w, blk, h) in b_next[slot]:
            read_half(tr, w, blk, h)
    assert not a_next and tr.q[-4:] == [("B", 1), ("B", 1), ("B", 0), ("B", 0)]
    e(f'"s_add_u32 s{S_KA}, s{S_KA}, 128')
    e(f'"s_add_u32 s{S_KB}, s{S_KB}, 128')
    e(f'"s_xor_b32 s{S_LDS}, s{S_LDS}, 0x10000')
    e(f'"s_add_u32 s{S_IT}, s{S_IT}, 1')
    e(f'"s_cmp_lt_u32 s{S_IT}, %[n]')
    e('"s_cbranch_scc1 L_sk_loop%=')
    e('"s_waitcnt vmcnt(0) lgkmcnt(0)')
    for _ in range(3):
        e('"s_nop 7')
    return L


def store_text(ii0, ii1, scaled):
    """Epilogue for block rows ii0 .. ii1 - 1 of the wave's 128 x 128 result that leaves the two stages alone: lane l
    of block (ii, j) holds row 16 ii + l % 16, columns 16 j + 4 (l / 16) .. + 3 in a[(8 ii + j) 4 .. + 3].  Per block
    row the 32 values become 16 registers of 16-bit pairs (CVT = the packing conversion of C's type, round to nearest
    even), go through a patch of 16 rows x 272 bytes that the wave owns behind the stages (rows padded by 16 bytes:
    the 8-byte writes of a half-wave and the 16-byte reads of a quarter-wave each hit every bank once) and leave as
    four 16-byte stores of whole 256-byte row pieces.  %[wr] / %[rd] = the lane's write / read address in the patch,
    %[voff] = its byte offset in the wave's block of C (row l / 16, columns 8 (l % 16) ..), s83 / s84 / s85 / s87 the
    offsets of rows 0-3 / 4-7 / 8-11 / 12-15 of the block row (%[rowstep] = 16 rows of C, %[q1] = 4 rows); rows past M
    lie beyond the descriptor's range and are dropped.  The conversions of block row ii + 1 overlap the trip of block
    row ii through the patch.  scaled: the fp32 sums are multiplied by %[alpha] first (one-byte operands)."""
    L = []
    e = L.append
    SO = (S_T, S_OOB, S_M0, S_T2)     # s83, s84, s85, s87
    e(f'"s_mul_i32 s{SO[0]}, %[rowstep], {ii0}')
    for k in range(1, 4):
        e(f'"s_add_u32 s{SO[k]}, s{SO[k - 1]}, %[q1]')

    def convert(ii):
        rd = 128 if (ii - ii0) % 2 == 0 else 192          # 32 fp32 values, then 16 registers of pairs behind them
        for r in range(32):
            e(f'"v_accvgpr_read_b32 v{rd + r}, a{ii * 32 + r}')
        if scaled:
            for r in range(32):
                e(f'"v_mul_f32 v{rd + r}, %[alpha], v{rd + r}')
        for q in range(16):
            e(f'CVT " v{rd + 32 + q}, v{rd + 2 * q}, v{rd + 2 * q + 1}')
        return rd + 32

    def out_regs(ii):
        return 176 if (ii - ii0) % 2 == 0 else 240        # the four 16-byte pieces read back from the patch

    def stores(ii):
        for k in range(4):
            e(f'"buffer_store_dwordx4 v[{out_regs(ii) + 4 * k}:{out_regs(ii) + 4 * k + 3}], %[voff], %[rsc], s{SO[k]} offen')
        for k in range(4):
            e(f'"s_add_u32 s{SO[k]}, s{SO[k]}, %[rowstep]')

    pk = convert(ii0)
    for ii in range(ii0, ii1):
        e('"s_waitcnt lgkmcnt(0)')                          # the reads of the previous block row have left the patch
        for j in range(8):
            e(f'"ds_write_b64 %[wr], v[{pk + 2 * j}:{pk + 2 * j + 1}] offset:{32 * j}')
        if ii > ii0:
            stores(ii - 1)
        if ii + 1 < ii1:
            pk = convert(ii + 1)
        e('"s_waitcnt lgkmcnt(0)')                          # the writes have landed (the wave's own, in order)
        for k in range(4):
            e(f'"ds_read_b128 v[{out_regs(ii) + 4 * k}:{out_regs(ii) + 4 * k + 3}], %[rd] offset:{1088 * k}')
    e('"s_waitcnt lgkmcnt(0)')
    stores(ii1 - 1)
    return L


def emit_macro(name, params, lines):
    print(f"#define {name}{params} \\")
    for text in lines:
        print(f"  {text}\\n\\t\" \\")
    print("  \"\"")


def main():
    print("// Generated by gen_tile_asm.py -- do not edit; see that file for the register plan and the schedule.")
    print("// SK_TILE_ASM_LOADS / _LOADS_NN: the 16 loads of one stage.  SK_TILE_ASM_LOOP(MF) / _LOOP_NN(MF): the loop for the")
    print("// NT / NN layout, MF = the MFMA mnemonic as a string literal.  SK_TILE_ASM_LOOP_F8(MF, MOD): fp8 operands, MOD =")
    print("// the format modifiers of the MFMA (\"\" for e4m3).  SK_TILE_ASM_STORE_x(CVT): the epilogue that leaves the stages alone.")
    print("#pragma once")
    emit_macro("SK_TILE_ASM_LOADS", "", stage_loads_text(False))
    emit_macro("SK_TILE_ASM_LOADS_NN", "", stage_loads_text(True))
    emit_macro("SK_TILE_ASM_LOOP", "(MF)", loop_text(False))
    emit_macro("SK_TILE_ASM_LOOP_NN", "(MF)", loop_text(True))
    emit_macro("SK_TILE_ASM_LOOP_F8", "(MF, MOD)", loop_text_f8())
    for name, (ii0, ii1) in (("ALL", (0, 8)), ("HALF0", (0, 4)), ("HALF1", (4, 8))):
        emit_macro(f"SK_TILE_ASM_STORE_{name}", "(CVT)", store_text(ii0, ii1, False))
        emit_macro(f"SK_TILE_ASM_STORE_{name}_SCALED", "(CVT)", store_text(ii0, ii1, True))
    clob = [f'"a{r}"' for r in range(256)] + [f'"v{r}"' for r in range(120, 256)] + [f'"s{r}"' for r in range(80, 88)]
    print("#define SK_TILE_ASM_CLOBBERS \\")
    for k in range(0, len(clob), 16):
        tail = ", \\" if k + 16 < len(clob) else ""
        print("  " + ", ".join(clob[k:k + 16]) + tail)


if __name__ == "__main__":
    main()
