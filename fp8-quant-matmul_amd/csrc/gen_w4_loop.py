#!/usr/bin/env python3
"""Writes w4_loop.inc: the K-block loop of the one-wave-per-SIMD tile kernel
(k_tile_persistent.hip, four waves of 128 x 96 each on a 256 x 192 tile) as register-exact assembly.

Why assembly, and why generated: with one wave per SIMD nobody else fills the issue slots, so the
order of every instruction matters, and the wave needs all 512 registers in a fixed arrangement
(running sums and block sums in v, operand fragments in a); left to the register allocator, the
running sums wander between the two register files.  The text names physical registers, which the
preprocessor cannot compute, hence this script.   python3 gen_w4_loop.py > w4_loop.inc

Register map of a wave
    v[16q : 16q+15]   q = 0..11   running sums of patch q = jj * 4 + i  (i: 32 rows of m, jj: 32 columns of n)
    v192, v193                    LDS read addresses (A fragments, B fragments)
    v[194:197]                    a_scale of the block, one value per patch row i
    v198, v199                    the two b_scale values of the block (as read from LDS)
    v200                          scale of the fold in progress (carried from block to block)
    v[201:223]                    the compiler's (operands of the statement)
    v[224:239], v[240:255]        block sums, set 0 / set 1 (patch p uses set p & 1)
    a[8f : 8f+7]      f = 0..13   operand fragments: A(i, ks) = 2i + ks, B(jj, ks) = 8 + 2jj + ks
    s[84:93]                      scratch scalars of the loop

Schedule of one K block (MFMA g = 2p + ks; "gap g" = what is issued behind it)
    * patches column by column (jj outer); the fold of the patch before (16 FMAs: sums += scale *
      block sums) rides in this patch's two gaps, FOLD_EVEN of them in the first, after that gap's
      memory instructions (its block sums are only one MFMA old there);
    * columns 0..NJ-2: the gaps fetch the next column's B fragments; gap 0 also fetches the scales;
    * before the last column: wait for this wave's copies of the next block, barrier;
    * last column: behind MFMA g the fragment it has just read for the last time is refilled from the
      next block (other ring slot), the first gaps also fetch the next block's B(0, *), and the copy
      instructions of the block after next go out into the slot just freed.
LDS waits: reads return in order, so "at most N younger operations outstanding" (s_waitcnt lgkmcnt(N),
N <= 15) is exact; N is derived below from the order of issue.  An MFMA's result may be read by an
ordinary instruction MFMA_RESULT_SLOTS instructions later at the earliest (no interlock; the value is
what the compiler pads a 16-pass MFMA with on this target): the FMAs of an even gap are padded with
s_nop up to that distance, counted on the emitted text.
"""
import sys

MI, NJ = 4, 3
NP = MI * NJ
GAPS_COL = 2 * MI
NG = GAPS_COL * NJ
RS = 256                    # LDS bytes per k-row of either matrix (BM = 256, BN = 192 -> 256)
MAT_A = 128 * RS
STAGE = 2 * MAT_A + 1024 + 256   # A rows, B rows, a_scale (1 KiB), b_scale (256 B)
NCOPY_AB = 8                # copy instructions per wave and matrix (128 rows * 256 B / 4 waves / 1 KiB)
MFMA_RESULT_SLOTS = 20
REFILL_SLOTS = 8             # instructions between an MFMA and a read that overwrites one of its operands
FOLD_EVEN = 4               # FMAs of a fold placed in the even gap (the rest in the odd one)
SCALE_OPS = 4
BLK = (224, 240)
V_ADDR_A, V_ADDR_B, V_SA, V_SB_LO, V_SB_HI, V_SC = 192, 193, 194, 198, 199, 200
S_SO, S_SO_NEXT, S_M0BASE, S_SOFF, S_SBLO, S_SBHI, S_SBJ, S_T0, S_T1 = 84, 85, 86, 88, 89, 90, 91, 92, 93


def frag_a(i, ks):
    return 2 * i + ks


def frag_b(jj, ks):
    return 8 + 2 * jj + ks


def piece_reg(f, t):
    return f"a[{8 * f + 2 * t}:{8 * f + 2 * t + 1}]"


def piece_off(ks, t):
    return (ks * 64 + 8 * t) * RS


# ---- which LDS operations ride in which gap (program order inside the gap)
def b_pieces_before_barrier(c):
    """pieces (u = 4*ks + t) of the next column's B fragments fetched in gap c of a column"""
    return [2 * c, 2 * c + 1] if c < 2 else ([c + 2] if c < 6 else [])


def b0_pieces_behind_barrier(c):
    """pieces of the next block's B(0, *) fetched in gap c of the last column"""
    return [2 * c, 2 * c + 1] if c < 4 else []


def gap_ops(g):
    """LDS operations of gap g: ('S', n) scale read n, ('A', i, ks, t), ('B', jj, ks, t)"""
    jj, c = divmod(g, GAPS_COL)
    ops = []
    if g == 0:
        ops += [("S", s) for s in range(SCALE_OPS)]
    if jj < NJ - 1:
        ops += [("B", jj + 1, u // 4, u % 4) for u in b_pieces_before_barrier(c)]
    else:
        ops += [("A", c // 2, c % 2, t) for t in range(4)]
        ops += [("B", 0, u // 4, u % 4) for u in b0_pieces_behind_barrier(c)]
    return ops


def younger_ops(g, needed):
    """LDS operations issued after the youngest of `needed` and before MFMA g (steady state)"""
    needed = set(needed)
    after = 0
    result = None
    for back in range(1, g + NG + 1):
        for op in reversed(gap_ops((g - back) % NG)):
            if op in needed:
                if result is None:
                    result = after
                needed.discard(op)
            after += 1
        if not needed:
            return result
    raise AssertionError(f"MFMA {g}: {needed} never fetched")


def mfma_wait(g):
    p, ks = divmod(g, 2)
    jj, i = divmod(p, MI)
    need = [("A", i, ks, t) for t in range(4)] + [("B", jj, ks, t) for t in range(4)]
    return min(15, younger_ops(g, need))


def scale_wait(g):
    return min(15, younger_ops(g, [("S", s) for s in range(SCALE_OPS)]))


# ---- text
class Asm:
    def __init__(self):
        self.lines = []
        self.skippable = set()   # indices of instructions a taken branch jumps over

    def __call__(self, text, skippable=False):
        if skippable:
            self.skippable.add(len(self.lines))
        self.lines.append(text)

    def slots_since(self, start):
        """instruction slots surely spent by lines[start:]: labels and skippable lines count nothing,
        s_nop N counts N + 1"""
        n = 0
        for k in range(start, len(self.lines)):
            ln = self.lines[k]
            if ln.endswith(":") or k in self.skippable:
                continue
            n += int(ln.split()[1]) + 1 if ln.startswith("s_nop") else 1
        return n

    def string(self, indent):
        pad = " " * indent
        return "\n".join(f'{pad}"{ln}\\n\\t"' for ln in self.lines)


def copy_parts(q, c_first):
    """copy instruction q of the block after next, into the slot of the current block, as
    (lines up to and including the one that sets M0, lines from the load on).  One instruction must
    lie between the write of M0 and the load: the caller puts an LDS read there, or s_nop."""
    head, tail = [], []
    mat, qq = divmod(q, NCOPY_AB)
    m = "ab"[mat]
    if qq == 0:
        if mat == 0 and c_first:
            head.append(f"s_add_u32 s{S_M0BASE}, s{S_SO}, %[lds_wave]")
        head.append(f"s_mov_b32 s{S_SOFF}, %[off_{m}]")
    head.append(f"s_add_u32 m0, s{S_M0BASE}, {mat * MAT_A + qq * 1024}")
    tail.append(f"buffer_load_dwordx4 %[voff_{m}{qq & 1}], %[rsrc_{m}], s{S_SOFF} offen lds")
    if qq & 1:
        tail.append(f"s_add_u32 s{S_SOFF}, s{S_SOFF}, %[ld8_{m}]")
    return head, tail


def scale_copy(a):
    """wave 0 brings the block's a_scale (16 bytes per lane), wave 1 its b_scale (4 bytes per lane)"""
    a("s_cmp_lg_u32 %[scale_kind], 0")
    a("s_cbranch_scc1 .Lw4_no_as_%=")
    a(f"s_add_u32 m0, s{S_SO}, %[lds_scale]", True)
    a("s_nop 0", True)
    a("buffer_load_dwordx4 %[voff_sc], %[rsrc_sc], %[off_sc] offen lds", True)
    a(".Lw4_no_as_%=:")
    a("s_cmp_lg_u32 %[scale_kind], 1")
    a("s_cbranch_scc1 .Lw4_no_bs_%=")
    a(f"s_add_u32 m0, s{S_SO}, %[lds_scale]", True)
    a("s_nop 0", True)
    a("buffer_load_dword %[voff_sc], %[rsrc_sc], %[off_sc] offen lds", True)
    a(".Lw4_no_bs_%=:")


def fold_part(a, q, d, lo, hi):
    """elements lo .. hi-1 of: sums of patch q += scale * block sums in set d"""
    for r in range(lo, hi):
        a(f"v_fmac_f32 v{16 * q + r}, v{V_SC}, v{BLK[d] + r}")


def lds_read_lines(op, jj):
    """instructions of one LDS operation of a gap in column jj"""
    if op[0] == "S":
        n = op[1]
        if n == 0:
            return [f"v_add_u32 v{V_SB_LO}, s{S_SO}, %[vaddr_s]",
                    f"ds_read2_b32 v[{V_SA}:{V_SA + 1}], v{V_SB_LO} offset0:0 offset1:32"]
        if n == 1:
            return [f"ds_read2_b32 v[{V_SA + 2}:{V_SA + 3}], v{V_SB_LO} offset0:64 offset1:96"]
        reg, name = (V_SB_LO, "sb_lo") if n == 2 else (V_SB_HI, "sb_hi")
        return [f"s_add_u32 s{S_T0}, s{S_SO}, %[lds_{name}]", f"v_mov_b32 v{reg}, s{S_T0}",
                f"ds_read_b32 v{reg}, v{reg}"]
    if op[0] == "B":
        _, bj, bks, bt = op
        src = S_SO_NEXT if jj == NJ - 1 else S_SO
        pre = [f"v_add_u32 v{V_ADDR_B}, s{src}, %[vbase_b{bj}]"] if (bks, bt) == (0, 0) else []
        return pre + [f"ds_read_b64_tr_b8 {piece_reg(frag_b(bj, bks), bt)}, v{V_ADDR_B} offset:{piece_off(bks, bt)}"]
    _, ai, aks, at = op
    pre = [f"v_add_u32 v{V_ADDR_A}, s{S_SO_NEXT}, %[vbase_a{ai}]"] if (aks, at) == (0, 0) else []
    return pre + [f"ds_read_b64_tr_b8 {piece_reg(frag_a(ai, aks), at)}, v{V_ADDR_A} offset:{piece_off(aks, at)}"]


def k_block(a, slots_before_first_fold):
    """one K block; slots_before_first_fold = instruction slots between the previous block's last MFMA
    and this block's first instruction (the loop's tail).  Returns the slots behind this block's last MFMA."""
    a(f"s_mov_b32 s{S_SO}, %[slot_off]")
    a(f"s_sub_u32 s{S_SO_NEXT}, {STAGE}, s{S_SO}")
    block_start = len(a.lines) - 2
    per_gap = -(-(2 * NCOPY_AB + 1) // GAPS_COL)
    last_mfma = None   # index of the line of the MFMA before the current one
    this_mfma = None
    for p in range(NP):
        jj, i = divmod(p, MI)
        pq = (p - 1) % NP          # the patch whose fold rides on this patch's MFMAs
        pj = pq // MI
        if p == 1:
            a(f"s_waitcnt lgkmcnt({scale_wait(2)})")
            a(f"v_readfirstlane_b32 s{S_SBLO}, v{V_SB_LO}")
            a(f"v_readfirstlane_b32 s{S_SBHI}, v{V_SB_HI}")
        if p >= 1 and (p - 1) % MI == 0:
            # the b_scale value of column pj: hi where the column lies in the wave's second 128-block
            a(f"s_and_b32 s{S_T0}, s{S_SBHI}, %[hi_mask{pj}]")
            a(f"s_andn2_b32 s{S_T1}, s{S_SBLO}, %[hi_mask{pj}]")
            a(f"s_or_b32 s{S_SBJ}, s{S_T0}, s{S_T1}")
        if p >= 1:
            a(f"v_mul_f32 v{V_SC}, s{S_SBJ}, v{V_SA + pq % MI}")
        if jj == NJ - 1 and i == 0:
            a("s_waitcnt vmcnt(0) lgkmcnt(0)")
            a("s_barrier")
        for ks in range(2):
            g = 2 * p + ks
            c = g % GAPS_COL
            d = p & 1
            a(f"s_waitcnt lgkmcnt({mfma_wait(g)})")
            last_mfma, this_mfma = this_mfma, len(a.lines)
            a(f"v_mfma_f32_32x32x64_f8f6f4 v[{BLK[d]}:{BLK[d] + 15}], a[{8 * frag_b(jj, ks)}:{8 * frag_b(jj, ks) + 7}], "
              f"a[{8 * frag_a(i, ks)}:{8 * frag_a(i, ks) + 7}], {'0' if ks == 0 else f'v[{BLK[d]}:{BLK[d] + 15}]'}")
            # ---- gap g.  Last column: the copies first (something must sit between the write of M0
            # and the load: a B read, else s_nop); the reads that refill the A fragment this MFMA is
            # reading come late in the gap (REFILL_SLOTS behind the MFMA at least, on top of the LDS
            # round trip).  FMAs: last in an even gap (their block sums are one MFMA old), before the
            # refill in an odd one.
            ops = gap_ops(g)
            b_reads = [ln for op in ops if op[0] != "A" for ln in lds_read_lines(op, jj)]
            a_reads = [ln for op in ops if op[0] == "A" for ln in lds_read_lines(op, jj)]
            if jj == NJ - 1:
                for q in range(per_gap * c, min(per_gap * (c + 1), 2 * NCOPY_AB + 1)):
                    if q == 2 * NCOPY_AB:
                        scale_copy(a)
                        continue
                    head, tail = copy_parts(q, c == 0)
                    for ln in head:
                        a(ln)
                    if b_reads:
                        a(b_reads.pop(0))
                        if a.lines[-1].startswith("v_add_u32"):   # the add that feeds the read: take both
                            a(b_reads.pop(0))
                    else:
                        a("s_nop 0")
                    for ln in tail:
                        a(ln)
            for ln in b_reads:
                a(ln)
            if ks == 1:
                fold_part(a, pq, (p + 1) & 1, FOLD_EVEN, 16)
            if a_reads:
                spent = a.slots_since(this_mfma + 1)
                if spent < REFILL_SLOTS:
                    a(f"s_nop {REFILL_SLOTS - spent - 1}")
                for ln in a_reads:
                    a(ln)
            if ks == 0:
                # these FMAs read what the MFMA before this one has written
                if last_mfma is None:
                    spent = slots_before_first_fold + a.slots_since(block_start)
                else:
                    spent = a.slots_since(last_mfma + 1)
                if spent < MFMA_RESULT_SLOTS:
                    a(f"s_nop {MFMA_RESULT_SLOTS - spent - 1}")
                fold_part(a, pq, (p + 1) & 1, 0, FOLD_EVEN)
    # scale of the last patch's fold, which rides on the next block's first MFMAs
    a(f"v_mul_f32 v{V_SC}, s{S_SBJ}, v{V_SA + MI - 1}")
    for m in ("a", "b", "sc"):
        a(f"s_add_u32 %[off_{m}], %[off_{m}], %[str_{m}]")
    a(f"s_xor_b32 %[slot_off], %[slot_off], {STAGE}")
    return this_mfma


def verify_distances(a):
    """The two hazards the loop keeps by counting instruction slots, checked on the emitted text over two
    rounds of the loop: a VALU read of a block sum lies at least MFMA_RESULT_SLOTS behind the MFMA that
    wrote it last, and a fragment read that overwrites an a-register lies at least REFILL_SLOTS behind the
    last MFMA that reads it.  (Both distances count from the MFMA's issue, as the schedule does.)"""
    import re
    first = a.lines.index(".Lw4_block_%=:")
    body = [(k, ln) for k, ln in enumerate(a.lines) if k > first]
    seq = body + body          # the second round sees the first round's MFMAs behind it
    cost = []                  # slots of each entry of seq
    for k, ln in seq:
        if ln.endswith(":") or k in a.skippable:
            cost.append(0)
        else:
            cost.append(int(ln.split()[1]) + 1 if ln.startswith("s_nop") else 1)
    mfma = re.compile(r"v_mfma\S* v\[(\d+):(\d+)\], a\[(\d+):(\d+)\], a\[(\d+):(\d+)\]")
    fmac = re.compile(r"v_fmac_f32 v\d+, v\d+, v(\d+)$")
    read = re.compile(r"ds_read_b64_tr_b8 a\[(\d+):(\d+)\]")
    checked = 0
    for pos in range(len(body), len(seq)):
        ln = seq[pos][1]
        need = None
        m = fmac.match(ln)
        if m and BLK[0] <= int(m.group(1)) < BLK[1] + 16:
            reg = int(m.group(1))
            need = (MFMA_RESULT_SLOTS, lambda mm: int(mm.group(1)) <= reg <= int(mm.group(2)))
        m = read.match(ln)
        if m:
            lo, hi = int(m.group(1)), int(m.group(2))
            need = (REFILL_SLOTS, lambda mm: any(int(mm.group(x)) <= hi and lo <= int(mm.group(x + 1)) for x in (3, 5)))
        if need is None:
            continue
        slots = 0
        for back in range(pos - 1, -1, -1):
            mm = mfma.match(seq[back][1])
            if mm and need[1](mm):
                assert slots >= need[0], f"'{ln}' is {slots} slots behind '{seq[back][1]}', needs {need[0]}"
                checked += 1
                break
            slots += cost[back]
        else:
            raise AssertionError(f"no MFMA found behind '{ln}'")
    assert checked > 0


def emit_loop(out):
    def build(tail_slots):
        a = Asm()
        a("s_waitcnt lgkmcnt(0)")   # scalar loads of the code around return out of order: none may be in flight
        a(".Lw4_block_%=:")
        last = k_block(a, tail_slots)
        a("s_sub_u32 %[count], %[count], 1")
        a("s_cmp_lg_u32 %[count], 0")
        a("s_cbranch_scc1 .Lw4_block_%=")
        return a, a.slots_since(last + 1)

    _, tail_slots = build(0)
    a, check = build(tail_slots)
    assert check == tail_slots, "the padding of the first gap changed the tail it was computed from"
    verify_distances(a)
    w = out.append
    w("// `count` (>= 1) K blocks of the current tile: MFMAs, folds, fragment reads, and the copies of the")
    w("// stream's next `count` blocks (offsets off_* advance by str_* per block; a stream that has run dry")
    w("// passes offsets outside its buffers).  On entry the fragments of the first block are in (or on their")
    w("// way into) a[0:111] in the order w4_first_reads issues them; on exit those of the block after the")
    w("// last one are.  slot_off = LDS byte offset of the ring slot of the block multiplied first (0 or")
    w(f"// {STAGE}), toggled per block.  scale_kind: 0 = this wave copies a_scale, 1 = b_scale, else none.")
    w("__device__ __forceinline__ void w4_k_blocks(")
    w("    v32f& sums0, v32f& sums1, v32f& sums2, v32f& sums3, v32f& sums4, v32f& sums5, v32f& blk,")
    w("    v32i& frag0, v32i& frag1, v32i& frag2, v16i& frag3, float& scale_carry,")
    w("    uint32_t vbase_a0, uint32_t vbase_a1, uint32_t vbase_a2, uint32_t vbase_a3, uint32_t vbase_b0,")
    w("    uint32_t vbase_b1, uint32_t vbase_b2, uint32_t vaddr_s, uint32_t voff_a0, uint32_t voff_a1,")
    w("    uint32_t voff_b0, uint32_t voff_b1, uint32_t voff_sc, v4i rsrc_a, v4i rsrc_b, v4i rsrc_sc,")
    w("    uint32_t& off_a, uint32_t& off_b, uint32_t& off_sc, uint32_t str_a, uint32_t str_b, uint32_t str_sc,")
    w("    uint32_t ld8_a, uint32_t ld8_b, uint32_t& slot_off, uint32_t lds_wave, uint32_t lds_scale,")
    w("    uint32_t scale_kind, uint32_t lds_sb_lo, uint32_t lds_sb_hi, uint32_t hi_mask0, uint32_t hi_mask1,")
    w("    uint32_t hi_mask2, uint32_t& count)")
    w("{")
    w("    asm volatile(")
    w(a.string(8))
    w('        : "+{v[0:31]}"(sums0), "+{v[32:63]}"(sums1), "+{v[64:95]}"(sums2), "+{v[96:127]}"(sums3),')
    w('          "+{v[128:159]}"(sums4), "+{v[160:191]}"(sums5), "+{v[224:255]}"(blk), "+{a[0:31]}"(frag0),')
    w('          "+{a[32:63]}"(frag1), "+{a[64:95]}"(frag2), "+{a[96:111]}"(frag3), "+{v200}"(scale_carry),')
    w('          [off_a] "+s"(off_a), [off_b] "+s"(off_b), [off_sc] "+s"(off_sc), [slot_off] "+s"(slot_off),')
    w('          [count] "+s"(count)')
    w('        : [vbase_a0] "v"(vbase_a0), [vbase_a1] "v"(vbase_a1), [vbase_a2] "v"(vbase_a2), [vbase_a3] "v"(vbase_a3),')
    w('          [vbase_b0] "v"(vbase_b0), [vbase_b1] "v"(vbase_b1), [vbase_b2] "v"(vbase_b2), [vaddr_s] "v"(vaddr_s),')
    w('          [voff_a0] "v"(voff_a0), [voff_a1] "v"(voff_a1), [voff_b0] "v"(voff_b0), [voff_b1] "v"(voff_b1),')
    w('          [voff_sc] "v"(voff_sc), [rsrc_a] "s"(rsrc_a), [rsrc_b] "s"(rsrc_b), [rsrc_sc] "s"(rsrc_sc),')
    w('          [str_a] "s"(str_a), [str_b] "s"(str_b), [str_sc] "s"(str_sc), [ld8_a] "s"(ld8_a), [ld8_b] "s"(ld8_b),')
    w('          [lds_wave] "s"(lds_wave), [lds_scale] "s"(lds_scale), [scale_kind] "s"(scale_kind),')
    w('          [lds_sb_lo] "s"(lds_sb_lo), [lds_sb_hi] "s"(lds_sb_hi), [hi_mask0] "s"(hi_mask0),')
    w('          [hi_mask1] "s"(hi_mask1), [hi_mask2] "s"(hi_mask2)')
    w('        : "memory", "scc", "v192", "v193", "v194", "v195", "v196", "v197", "v198", "v199",')
    w('          "s84", "s85", "s86", "s87", "s88", "s89", "s90", "s91", "s92", "s93");')
    w("}")


def emit_first_reads(out):
    a = Asm()
    for c in range(GAPS_COL):
        for op in gap_ops((NJ - 1) * GAPS_COL + c):
            if op[0] == "A":
                _, ai, aks, at = op
                a(f"ds_read_b64_tr_b8 {piece_reg(frag_a(ai, aks), at)}, %[vbase_a{ai}] offset:{piece_off(aks, at)}")
            else:
                _, bj, bks, bt = op
                a(f"ds_read_b64_tr_b8 {piece_reg(frag_b(bj, bks), bt)}, %[vbase_b0] offset:{piece_off(bks, bt)}")
    w = out.append
    w("")
    w("// the fragments of the very first block, from ring slot 0, in the order the last column of a block")
    w("// before would have fetched them (the counted waits of w4_k_blocks rely on that order)")
    w("__device__ __forceinline__ void w4_first_reads(v32i& frag0, v32i& frag1, v32i& frag2, v16i& frag3,")
    w("                                               uint32_t vbase_a0, uint32_t vbase_a1, uint32_t vbase_a2,")
    w("                                               uint32_t vbase_a3, uint32_t vbase_b0)")
    w("{")
    w("    asm volatile(")
    w(a.string(8))
    w('        : "+{a[0:31]}"(frag0), "+{a[32:63]}"(frag1), "+{a[64:95]}"(frag2), "+{a[96:111]}"(frag3)')
    w('        : [vbase_a0] "v"(vbase_a0), [vbase_a1] "v"(vbase_a1), [vbase_a2] "v"(vbase_a2), [vbase_a3] "v"(vbase_a3),')
    w('          [vbase_b0] "v"(vbase_b0)')
    w('        : "memory");')
    w("}")


def emit_drain(out):
    a = Asm()
    a("s_nop 15")
    a(f"s_nop {MFMA_RESULT_SLOTS - 16 - 1}")
    fold_part(a, NP - 1, (NP - 1) & 1, 0, 16)
    w = out.append
    w("")
    w("// the fold that a tile's last block leaves behind (its last patch, scale in scale_carry), behind")
    w("// the distance an MFMA result needs")
    w("__device__ __forceinline__ void w4_last_fold(v32f& sums5, v32f& blk, float scale_carry)")
    w("{")
    w("    asm volatile(")
    w(a.string(8))
    w('        : "+{v[160:191]}"(sums5), "+{v[224:255]}"(blk)')
    w('        : "{v200}"(scale_carry));')
    w("}")


def main():
    out = ["// GENERATED by gen_w4_loop.py -- do not edit; schedule and register map are documented there.",
           f"// STAGE = {STAGE} bytes per ring slot; MFMA waits: " + " ".join(str(mfma_wait(g)) for g in range(NG)),
           ""]
    emit_loop(out)
    emit_first_reads(out)
    emit_drain(out)
    sys.stdout.write("\n".join(out) + "\n")


if __name__ == "__main__":
    main()
