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

  SK_TILE_ASM_LOADS*   the 16 direct-to-LDS loads of one 64 KB stage (8 row groups of A, 8 of B per wave), or
                       (_EARLY) the half of them the loop does not send itself.  A segment starts with the loads of its
                       first stage and the early loads of its second; the first stage of the NEXT segment is requested
                       before the epilogue of the current one, so that its latency hides behind the stores of C.
  SK_TILE_ASM_LOOP*    zero the accumulators, wait for the first stage, run the K loop, drain.
  SK_TILE_ASM_STORE*   the epilogue of a tile that needs no edge handling: accumulators -> 16-bit pairs -> a small
                       per-wave patch of LDS behind the stages -> 16-byte stores of whole row pieces.  The stages are
                       not touched, which is what allows the next segment's loads to be in flight.

One iteration of the 16-bit loop is two blocks of 64 MFMAs, one per K-step of 32, built alike (loop_text has the
details).  The loads of a stage come in two halves: the row groups that hold blocks 0-3 of the wave tiles (EARLY) and
those that hold blocks 4-7 (LATE).  The MFMAs of a block run quadrant by quadrant, so the late fragments are needed
only from the 17th instruction on and are read at the top of their own block; everything a block reads at its top
was loaded a half-stage later and is overwritten a half-stage later than the rest.  That shifts the two halves of a
stage by one block against each other, and every block carries eight loads.  Counters on 8192^3 (SQ_BUSY_CU_CYCLES,
SQ_VMEM_TA_ADDR_FIFO_FULL): with all 16 loads of an iteration in one block, the four waves' 64 KB keep the CU's one
address unit busy for that whole block, a wave whose load finds the address queue full cannot issue its next MFMA
either, the waves drift apart and the barrier makes every wave pay the slowest one's delay -- removing the barrier
(wrong results, timing only) gave +22 % on zero operands, removing the wait for the loads nothing; with eight loads
per block the queue-full cycles fall to a quarter and the time by 10 % (zero operands) / 3 % (random operands, where
the clock is set by the power drawn).  Placing the loads of the four waves in different gaps, or earlier in their
block, or the reads earlier, changed nothing measurable.
Riders are dealt out ONE GROUP PER MFMA GAP (a gap is the 16 cycles an MFMA occupies the matrix pipe; the wave issues
about one other instruction per four cycles in it): with the four instructions of a load in one gap every load cost
~10 cycles of matrix-pipe time.  An MFMA that waits for a fragment waits only for the reads it needs (the waits are
computed from the issue order: LDS reads return in order).
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

# Row groups of a wave's eight per operand (group x holds rows 8 (wave + 4 x) .. + 7 of the tile's 256): the EARLY ones
# carry rows of blocks 0-3 of a wave's 128 rows, the LATE ones rows of blocks 4-7
EARLY_X, LATE_X = (0, 1, 4, 5), (2, 3, 6, 7)
TOP = 8     # gaps at the top of a block that carry the reads of the late fragments
LD_LAST, RD_LAST = 61, 53    # last gap of a block that may carry a load / a fragment read of the next K-step


def mfma_order():
    """the 8 x 8 blocks quadrant by quadrant -- (A 0-3, B 0-3), (A 0-3, B 4-7), (A 4-7, B 4-7), (A 4-7, B 0-3) -- so that
    the fragments of blocks 4-7 are needed only from the 17th (B) and the 33rd (A) instruction on; consecutive
    instructions share one operand"""
    def snake(rows, cols):
        out = []
        for n, i in enumerate(rows):
            out += [(i, j) for j in (cols if n % 2 == 0 else cols[::-1])]
        return out
    lo, hi = [0, 1, 2, 3], [4, 5, 6, 7]
    return snake(lo, lo) + snake(lo[::-1], hi) + snake(hi, hi) + snake(hi[::-1], lo[::-1])


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


def load_parts(x, nn, voa, vob, vob1, lds, ka, kb, prev=None):
    """load x of a stage: 0..7 row groups of A, 8..15 of B (a wave's groups are 4 KB apart in LDS).  Returns
    (instructions that go before the m0 write, the m0 write, the load); s[S_T] walks the global offsets of the
    groups -- `prev` is the group the walk comes from (None: x is the first of its operand in this sequence) --,
    `lds` is the stage's LDS address for this wave"""
    base, step, first = (ka, "%[gas", 0) if x < 8 else (kb, "%[gbs", 8)
    if prev is None:
        skip = x - first
        pre = [f'"s_mov_b32 s{S_T}, {base}'] if skip == 0 else [f'"s_add_u32 s{S_T}, {base}, {step}{skip}]']
    else:
        pre = [f'"s_add_u32 s{S_T}, s{S_T}, {step}{x - prev}]']
    pre = [t.replace("gas1]", "gas]").replace("gbs1]", "gbs]") for t in pre]
    lds_off = (x * 4096) if x < 8 else (32768 + (x - 8) * 4096)
    m0 = f'"s_add_u32 m0, {lds}, {lds_off}'
    if x < 8:
        ld = f'"buffer_load_dwordx4 {voa}, %[rsa], s{S_T} offen lds'
    else:
        ld = f'"buffer_load_dwordx4 {vob1 if (nn and x % 2 == 1) else vob}, %[rsb], s{S_T} offen lds'
    return pre, m0, ld


def load_sequence(xs, nn, voa, vob, vob1, lds, ka, kb):
    """load_parts for the groups xs (ascending; A before B), with the walk chained through them"""
    out, prev = [], None
    for x in xs:
        if prev is not None and (prev < 8) != (x < 8):
            prev = None
        out.append(load_parts(x, nn, voa, vob, vob1, lds, ka, kb, prev))
        prev = x
    return out


def early_groups(nn):
    """the loads that must have landed a block ahead of the others: rows of blocks 0-3 (NN: and all of B, whose loads
    fill whole K-rows)"""
    return list(EARLY_X) + ([8 + x for x in range(8)] if nn else [8 + x for x in EARLY_X])


def late_groups(nn):
    return list(LATE_X) + ([] if nn else [8 + x for x in LATE_X])


def stage_loads_text(nn, xs):
    """the loads xs of one stage, back to back (operands: the stage's LDS address, global offsets and lane offsets)"""
    L = []
    for pre, m0, ld in load_sequence(xs, nn, "%[voa]", "%[vob]", "%[vob1]", "%[lds]", "%[ga]", "%[gb]"):
        L += pre + [m0, '"s_nop 0', ld]
    return L


def offsets_for(nn, ahead):
    """v120 / v121 = the lane offsets, pushed out of range if iteration it + ahead is past the segment"""
    out = [f'"s_add_u32 s{S_T2}, s{S_IT}, {ahead}', f'"s_cmp_lt_u32 s{S_T2}, %[n]', f'"s_cselect_b32 s{S_OOB}, 0, 0x80000000',
           f'"v_or_b32 v{VOA}, s{S_OOB}, %[voa]', f'"v_or_b32 v{VOB}, s{S_OOB}, %[vob]']
    if nn:
        out.append(f'"v_or_b32 v{VOB1}, s{S_OOB}, %[vob1]')
    return out


def zero_accumulators(L):
    for r in range(256):
        L.append(f'"v_accvgpr_write_b32 a{r}, 0')


def spread(plan, groups, first, last):
    """deals `groups` (lists of instruction texts) out over the free gaps among first .. last, in order and evenly"""
    free = [g for g in range(first, last + 1) if g not in plan]
    assert len(free) >= len(groups), (len(free), len(groups), first, last)
    for k, item in enumerate(groups):
        plan[free[(k * len(free)) // len(groups)]] = item


def loop_text(nn):
    """The loop for the NT (nn = False) or the NN layout.  The two blocks of an iteration are built alike; block b
    (K-step b of iteration `it`, fragment set b, stage cur = it % 2, nxt the other one):
      top      reads of the LATE fragments (blocks 4-7 of A and B) of set b from cur -- their rows were the last to
               be loaded and are the last to be overwritten
      riders   reads of the EARLY fragments of the next K-step into the other set (b = 0: K-step 1 from cur, b = 1:
               K-step 0 of it + 1 from nxt); eight loads (b = 0: the LATE row groups of it + 1 into nxt, b = 1: the
               EARLY row groups of it + 2 into cur); address flips and, in block 1, the loop's scalar state
      end      wait for the reads and for the eight loads issued a block earlier, barrier
    so every load has between one and two blocks to land, and each block sends the same number of loads."""
    L = []
    e = L.append
    kb_step = "%[kbs]" if nn else "128"
    order = mfma_order()
    n_early, n_late = len(early_groups(nn)), len(late_groups(nn))

    def mf(i, j, ab, bb):
        c = (8 * i + j) * 4
        return f'MF " a[{c}:{c + 3}], v[{bb + 4 * j}:{bb + 4 * j + 3}], v[{ab + 4 * i}:{ab + 4 * i + 3}], a[{c}:{c + 3}]'

    # fragment reads as (tags, texts); 16 rows of 128 bytes per block of A (NT: of B too)
    def read_a(i, kk):
        ab, addr = (A0, "%[ra0]") if kk == 0 else (A1, "%[ra1]")
        return ([("A", kk, i)], [f'"ds_read_b128 v[{ab + 4 * i}:{ab + 4 * i + 3}], {addr} offset:{i * 2048}'])

    def read_b(j, kk):
        bb = B0 if kk == 0 else B1
        if not nn:
            addr = "%[rb0]" if kk == 0 else "%[rb1]"
            return ([("B", kk, j)], [f'"ds_read_b128 v[{bb + 4 * j}:{bb + 4 * j + 3}], {addr} offset:{j * 2048}'])
        # NN: two halves of four K-rows each, issued together
        return ([("B", kk, j)] * 2,
                [f'"ds_read_b64_tr_b16 v[{bb + 4 * j + 2 * h}:{bb + 4 * j + 2 * h + 1}], %[rbt{j}] offset:{kk * 16384 + h * 2048}'
                 for h in range(2)])

    def early_reads(kk):    # in the order the first quadrant needs them
        return [read_a(0, kk)] + [read_b(j, kk) for j in range(4)] + [read_a(i, kk) for i in range(1, 4)]

    def late_reads(kk):     # B 4-7 are needed from the 17th MFMA on, A 4-7 from the 33rd
        return [read_b(j, kk) for j in range(4, 8)] + [read_a(i, kk) for i in range(4, 8)]

    def load_groups(xs):
        """loads as rider groups: the scalar instructions of a load share a gap, the load has its own"""
        groups = []
        for pre, m0, ld in load_sequence(xs, nn, f"v{VOA}", f"v{VOB}", f"v{VOB1}", f"s{S_LDS}", f"s{S_KA}", f"s{S_KB}"):
            groups += [(None, pre + [m0]), (None, [ld])]
        return groups

    def block(b, tr, plan, closing):
        ab, bb = (A0, B0) if b == 0 else (A1, B1)
        for m, (i, j) in enumerate(order):
            w = tr.wait_for({("A", b, i), ("B", b, j)})
            if w:
                e(w)
            e(mf(i, j, ab, bb))
            tags, texts = plan.get(m, (None, []))
            L.extend(texts)
            for t in tags or []:
                tr.issue(t)
        assert all(0 <= g < 64 for g in plan), sorted(plan)
        L.extend(closing)

    # ---- entry: accumulators to zero while the first stage is on its way; the loop's state: the loads of block 0 are
    # those of iteration 1, into the second stage
    zero_accumulators(L)
    e(f'"s_mov_b32 s{S_IT}, 0')
    e(f'"s_xor_b32 s{S_LDS}, %[lds], 0x10000')
    e(f'"s_add_u32 s{S_KA}, %[ga0], 128')
    e(f'"s_add_u32 s{S_KB}, %[gb0], {kb_step}')
    L.extend(offsets_for(nn, 1))
    # (the youngest vector memory operations are the early loads of the second stage; the first stage has landed)
    e(f'"s_waitcnt vmcnt({n_early})')
    e('"s_barrier')
    at_top = []
    for tags, texts in early_reads(0):
        L.extend(texts)
        at_top += tags
    e('"s_nop 7')   # accumulator writes above are long done; cheap insurance before the first MFMA
    flip = lambda reg: (None, [f'"v_xor_b32 {reg}, 0x10000, {reg}'])

    def body():
        e('"L_sk_loop%=:')
        # ---- block 0
        plan = {}
        for g, item in enumerate(late_reads(0)):
            plan[g] = item
        spread(plan, load_groups(late_groups(nn)), TOP, LD_LAST)
        spread(plan, early_reads(1), TOP, RD_LAST)
        # the addresses of set 0 move to the other stage behind the reads at the top (block 1 reads the early fragments
        # of the next iteration with them); NN: one register per block of B serves both K-steps -- those of blocks 0-3
        # flip between the early reads of block 0 and of block 1, those of blocks 4-7 behind the top reads of block 1
        spread(plan, [flip("%[ra0]")] + ([] if nn else [flip("%[rb0]")]), TOP, 63)
        # both ways into the loop: the early fragments of set 0 may still be in flight
        block(0, LdsTracker(at_top), plan,
              [f'"s_waitcnt vmcnt({n_late}) lgkmcnt(0)', '"s_barrier'])       # (the early loads, issued a block ago, have landed)

        # ---- block 1
        plan = {}
        for g, item in enumerate(late_reads(1)):
            plan[g] = item
        state = [(None, [f'"s_add_u32 s{S_KA}, s{S_KA}, 128', f'"s_add_u32 s{S_KB}, s{S_KB}, {kb_step}']),
                 (None, [f'"s_xor_b32 s{S_LDS}, s{S_LDS}, 0x10000', f'"s_add_u32 s{S_T2}, s{S_IT}, 2']),
                 (None, [f'"s_cmp_lt_u32 s{S_T2}, %[n]', f'"s_cselect_b32 s{S_OOB}, 0, 0x80000000'])]
        state += [(None, [t]) for t in offsets_for(nn, 2)[3:]]
        if nn:
            state += [flip(f"%[rbt{j}]") for j in range(4)]
        for g, item in enumerate(state):
            plan[TOP + g] = item
        after_state = TOP + len(state)
        plan[63] = (None, [f'"s_add_u32 s{S_IT}, s{S_IT}, 1'])
        spread(plan, load_groups(early_groups(nn)), after_state, LD_LAST)
        spread(plan, early_reads(0), after_state, RD_LAST)
        spread(plan, [flip("%[ra1]")] + ([flip(f"%[rbt{j}]") for j in range(4, 8)] if nn else [flip("%[rb1]")]), after_state, 62)
        block(1, LdsTracker(), plan,
              [f'"s_waitcnt vmcnt({n_early}) lgkmcnt(0)', '"s_barrier',           # (the late loads of iteration it + 1 have landed)
               f'"s_cmp_lt_u32 s{S_IT}, %[n]', '"s_cbranch_scc1 L_sk_loop%='])

    body()
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
        pre, m0, ld = load_parts(x, False, f"v{VOA}", f"v{VOB}", f"v{VOB1}", f"s{S_LDS}", f"s{S_KA}", f"s{S_KB}",
                                 None if x in (0, 8) else x - 1)
        L.extend(pre + [m0, '"s_nop 0', ld])

    zero_accumulators(L)
    e(f'"s_mov_b32 s{S_IT}, 0')
    e(f'"s_mov_b32 s{S_LDS}, %[lds]')
    e(f'"s_add_u32 s{S_KA}, %[ga0], 256')     # the loads in the loop start with iteration 2
    e(f'"s_add_u32 s{S_KB}, %[gb0], 256')
    e('"s_waitcnt vmcnt(16)')     # (the 16 youngest vector memory operations are the loads of the second stage)
    e('"s_barrier')
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
    emit_macro("SK_TILE_ASM_LOADS", "", stage_loads_text(False, range(16)))
    emit_macro("SK_TILE_ASM_LOADS_NN", "", stage_loads_text(True, range(16)))
    emit_macro("SK_TILE_ASM_LOADS_EARLY", "", stage_loads_text(False, early_groups(False)))
    emit_macro("SK_TILE_ASM_LOADS_EARLY_NN", "", stage_loads_text(True, early_groups(True)))
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
