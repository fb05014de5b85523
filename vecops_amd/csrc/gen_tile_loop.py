#!/usr/bin/env python3
"""Writes tile_loop_asm.inc: the K loop of the 256x256 workgroup tile on the 16x16 matrix instructions, as one
instruction stream (inline assembly text).

Why a written-out stream: a wavefront of this tile owns 128x128 of C = 64 accumulator quads = all 256 registers of
the accumulation half of the register file.  Through the compiler's builtins such a loop gets its accumulators
renamed on every trip and copied back at the loop's head; written out, every matrix instruction accumulates in
place, every LDS address is a base register plus an immediate, and the order of issue is exactly the one below.

One K tile (128 bytes of each operand row) = two k-steps of 64 matrix instructions.  The tile in LDS stage S:
  k-step 0   multiplies fragment set 0 and reads the fragments of k-step 1 (stage S) into set 1
  barrier    (every wavefront has read stage S for the last time; the next tile's loads have landed in stage S^1)
  k-step 1   multiplies set 1, reads the fragments of the next tile's k-step 0 (stage S^1) into set 0 and issues
             the loads (they write LDS themselves) of the tile after the next into stage S
On the last two trips the loads go out against a descriptor of no records: they fetch nothing.

Fragment registers are fixed (v128..v255: set s, A block i at v[128+64s+4i..], B block j at v[160+64s+4j..]); the
accumulators, addresses and descriptors are operands of the statement (see asm_k_loop in tile_gemm.h, which
documents each of them).

    python3 gen_tile_loop.py > tile_loop_asm.inc
"""
import os
import sys

# experiments (not for shipping: results are wrong without the waits): GEN_DROP=vmwait,barrier,dma,reads
DROP = set(filter(None, os.environ.get("GEN_DROP", "").split(",")))


def fa(s, i):
    return f"v[{128 + 64 * s + 4 * i}:{128 + 64 * s + 4 * i + 3}]"


def fb(s, j):
    return f"v[{160 + 64 * s + 4 * j}:{160 + 64 * s + 4 * j + 3}]"


def fb_half(s, j, h):
    r = 160 + 64 * s + 4 * j + 2 * h
    return f"v[{r}:{r + 1}]"


STAGE = 65536       # bytes of one LDS stage: 256 rows of A and 256 of B (either layout), 128 bytes each
B_TILE = 32768      # the B tile lies behind the A tile
PITCH_TR = 512      # bytes between the k rows of a B tile kept as it lies in memory ([k][n], 256 columns)


def fragment_reads(tr, st, ks, to_set):
    """The reads of k-step ks of stage st into fragment set to_set, in the order the matrix instructions consume
    them: A block 0, every B block, the other A blocks.  tr: False (B K-contiguous, swizzled rows of 128 bytes), True
    (B as [k][n], transposing reads) or "pk" (B prepacked and kept in its pack order: [panel of 32 rows][k-step of two
    chunks][chunk half][row][16 bytes]; a wavefront's column block j lies in its panel j / 2, rows 16 (j % 2) .. + 15,
    and the lane's part of the address - its chunk and row - is in the one base register)."""
    out = []

    def a_read(i):
        q = (2 * ks ^ i) & 3
        out.append(f"ds_read_b128 {fa(to_set, i)}, %[la{st}{q}] offset:{i * 2048}")

    def b_read(j):
        if tr == "pk":
            out.append(f"ds_read_b128 {fb(to_set, j)}, %[lb{st}0] offset:{(j >> 1) * 4096 + ks * 2048 + (j & 1) * 256}")
        elif tr:
            off = (j & 1) * 32 + ks * 32 * PITCH_TR
            out.append(f"ds_read_b64_tr_b16 {fb_half(to_set, j, 0)}, %[lb{st}{j >> 1}] offset:{off}")
            out.append(f"ds_read_b64_tr_b16 {fb_half(to_set, j, 1)}, %[lb{st}{j >> 1}] offset:{off + 4 * PITCH_TR}")
        else:
            q = (2 * ks ^ j) & 3
            out.append(f"ds_read_b128 {fb(to_set, j)}, %[lb{st}{q}] offset:{j * 2048}")

    a_read(0)
    for j in range(8):
        b_read(j)
    for i in range(1, 8):
        a_read(i)
    return out


def loads(tr, st):
    """The sixteen loads of one K tile into stage st, each as (instructions in front of a matrix instruction,
    instructions behind it): M0 is written one instruction ahead of the load that uses it."""
    out = []
    for p in range(8):
        out.append(([f"s_add_u32 m0, %[m0w], {st * STAGE + p * 4096}"],
                    [f"buffer_load_dwordx4 %[ra{p}], s[80:83], %[ka] offen lds"]))
    for p in range(8):
        m0 = f"s_add_u32 m0, %[m0w], {st * STAGE + B_TILE + p * 4096}"
        if tr is True:
            pre = [m0] if p == 0 else [m0, "s_add_u32 s88, s88, %[pb]"]
            if p == 0:
                pre.append("s_mov_b32 s88, %[kb]")
            out.append((pre, ["buffer_load_dwordx4 %[rb0], s[84:87], s88 offen lds"]))
        else:
            out.append(([m0], [f"buffer_load_dwordx4 %[rb{p}], s[84:87], %[kb] offen lds"]))
    return out


def spread(n_items, n_slots, first=0):
    """slot -> list of item indices: item r goes behind matrix instruction first + floor(r * n_slots / n_items)"""
    where = {}
    for r in range(n_items):
        where.setdefault(first + (r * n_slots) // n_items, []).append(r)
    return where


def k_tile(tr, st):
    out = []
    order = os.environ.get("GEN_ORDER", "a_outer")
    def mfma(x, s):
        # x-th instruction of the k-step -> (A block i, B block j)
        if order == "a_outer":      # A block fixed over eight instructions
            i, j = x // 8, x % 8
        elif order == "snake":      # the same, B blocks back and forth
            i = x // 8
            j = x % 8 if i % 2 == 0 else 7 - x % 8
        elif order == "b_outer":
            j, i = x // 8, x % 8
        c = i * 8 + j
        return f"MFMA %[c{c}], {fb(s, j)}, {fa(s, i)}, %[c{c}]"
    # fetch nothing once no tile is left to fetch: a descriptor of no records
    out += ["s_cmp_gt_i32 %[left], 0",
            "s_cselect_b32 s82, 0x7fffffff, 0",
            "s_cselect_b32 s86, 0x7fffffff, 0",
            "s_sub_u32 %[left], %[left], 1"]
    # k-step 0
    reads = fragment_reads(tr, st, 1, 1)
    at = spread(len(reads), 40)
    out.append("s_waitcnt lgkmcnt(0)")
    for x in range(64):
        out.append(mfma(x, 0))
        for r in at.get(x, []):
            out.append(reads[r])
    out += ["s_waitcnt lgkmcnt(0)" if "vmwait" in DROP else "s_waitcnt vmcnt(0) lgkmcnt(0)"]
    if "barrier" not in DROP:
        out.append("s_barrier")
    # k-step 1
    reads = fragment_reads(tr, st ^ 1, 0, 0)
    at = spread(len(reads), 24, first=1) if tr is not True else spread(len(reads), 36, first=1)
    ld = loads(tr, st)
    every = int(os.environ.get("GEN_LOAD_EVERY", "4"))
    ld_at = {every * i: i for i in range(16)}   # load i straddles matrix instruction every * i
    assert max(ld_at) < 64
    if "dma" in DROP:
        ld_at = {}
    for x in range(64):
        if x in ld_at:
            out += ld[ld_at[x]][0]
        out.append(mfma(x, 1))
        if x in ld_at:
            out += ld[ld_at[x]][1]
        for r in at.get(x, []):
            out.append(reads[r])
    if "kadvance" not in DROP:
        out += ["s_add_u32 %[ka], %[ka], 128", "s_add_u32 %[kb], %[kb], %[sb]"]
    if "reads" in DROP:
        out = [line for line in out if not line.startswith("ds_read")]
    return out


def loop(tr):
    out = []
    # descriptors into fixed scalar registers: word 2 (the record count) is switched inside the loop
    for w in range(4):
        out.append(f"s_mov_b32 s{80 + w}, %[da{w}]")
        out.append(f"s_mov_b32 s{84 + w}, %[db{w}]")
    out += fragment_reads(tr, 0, 0, 0)
    out.append("1:")
    out += ["s_cmp_lt_u32 %[n], 2", "s_cbranch_scc1 2f"]
    out += k_tile(tr, 0)
    out += k_tile(tr, 1)
    out += ["s_sub_u32 %[n], %[n], 2", "s_branch 1b", "2:"]
    out += ["s_cmp_eq_u32 %[n], 0", "s_cbranch_scc1 3f"]
    out += k_tile(tr, 0)
    out.append("3:")
    # every load has landed (the epilogue lays C out in LDS) and every matrix result is written before the
    # statement ends: the compiler does not know that these registers come out of the matrix pipe
    out += ["s_waitcnt vmcnt(0) lgkmcnt(0)", "s_nop 15", "s_nop 15"]
    return out


# ---- the 256 x 352 tile (int8): 8 x 11 accumulator quads per wavefront -------------------------------------
# A wavefront owns 128 rows x 176 columns: A blocks i = 0..7 (rows wm * 128 + 16 i), B blocks j = 0..10, which are
# the blocks 2 j + wn of the workgroup's 22 (interleaved, so that the LDS swizzle of a fragment read stays a base
# register plus a constant).  88 accumulator quads: 64 in accumulation registers, 24 in vector registers.  Fragment
# registers: A blocks single (v[128 + 4 i ..]), B blocks double (set s at v[160 + 44 s + 4 j ..]).
#   k-step 0 of a tile multiplies B set 0; it reads B set 1 (this tile's k-step 1) and, behind the last
#   instruction of each row of blocks, that row's A fragment of k-step 1 into the registers just freed.
#   The barrier stands one row into k-step 1 (the last of those reads has landed by then); behind it the loads of
#   the tile after the next go into this stage and the next tile's k-step 0 fragments are read from the other.
# A's descriptor carries the bytes the tile's rows really have (%[na]: rows past M fetch zeros instead of being clamped).
# LDS reads complete in order, so each matrix instruction waits for "at most N reads issued after the one I need":
# the generator follows the reads through two trips of the loop and writes the counted waits.
WIDE_FM, WIDE_FN = 8, 11
WIDE_STAGE = (256 + 352) * 128


def wide_fa(i):
    return f"v[{128 + 4 * i}:{128 + 4 * i + 3}]"


def wide_fb(s, j):
    return f"v[{160 + 44 * s + 4 * j}:{160 + 44 * s + 4 * j + 3}]"


class ReadTracker:
    """Counted LDS waits: reads are numbered in issue order; `done` = every read up to this number has landed."""

    def __init__(self):
        self.issued = 0
        self.done = 0
        self.last_write = {}   # register name -> number of the read that fills it

    def read(self, out, reg, text):
        out.append(text)
        self.issued += 1
        self.last_write[reg] = self.issued

    def need(self, out, regs):
        upto = max(self.last_write.get(r, 0) for r in regs)
        if upto > self.done:
            out.append(f"s_waitcnt lgkmcnt({min(self.issued - upto, 15)})")
            self.done = upto if self.issued - upto <= 15 else self.issued - 15

    def need_all(self, out):
        if self.issued > self.done:
            out.append("s_waitcnt lgkmcnt(0)")
            self.done = self.issued


def wide_k_tile(st, tr):
    out = []
    acc = lambda i, j: f"%[c{i * WIDE_FN + j}]"

    def a_read(i, ks, stage):
        q = (2 * ks ^ i) & 3
        tr.read(out, ("a", i), f"ds_read_b128 {wide_fa(i)}, %[la{stage}{q}] offset:{i * 2048}")

    def b_read(to_set, j, ks, stage):
        q = (ks ^ j) & 1
        tr.read(out, ("b", to_set, j), f"ds_read_b128 {wide_fb(to_set, j)}, %[lb{stage}{q}] offset:{j * 4096}")

    out += ["s_cmp_gt_i32 %[left], 0",
            "s_cselect_b32 s82, %[na], 0",
            "s_cselect_b32 s86, 0x7fffffff, 0",
            "s_sub_u32 %[left], %[left], 1"]
    loads = []
    for p in range(8):
        pre = [f"s_add_u32 m0, %[m0w], {st * WIDE_STAGE + p * 4096}"]
        pre.append("s_mov_b32 s88, %[ka]" if p == 0 else "s_add_u32 s88, s88, %[pa]")
        loads.append((pre, [f"buffer_load_dwordx4 %[ra{p & 1}], s[80:83], s88 offen lds"]))
    for p in range(11):
        loads.append(([f"s_add_u32 m0, %[m0w], {st * WIDE_STAGE + 32768 + p * 4096}"],
                      [f"buffer_load_dwordx4 %[rb{p}], s[84:87], %[kb] offen lds"]))
    x = 0
    for ks in range(2):
        for i in range(WIDE_FM):
            for j in range(WIDE_FN):
                load = None
                if ks == 1 and x >= 100 and (x - 100) % 4 == 0 and (x - 100) // 4 < len(loads):
                    load = loads[(x - 100) // 4]
                    out += load[0]
                tr.need(out, [("a", i), ("b", ks, j)])
                out.append(f"MFMA {acc(i, j)}, {wide_fb(ks, j)}, {wide_fa(i)}, {acc(i, j)}")
                if load:
                    out += load[1]
                if ks == 0:
                    # this tile's k-step 1: B set 1 early, A block i behind its row
                    if x % 3 == 0 and x // 3 < WIDE_FN:
                        b_read(1, x // 3, 1, st)
                    if j == WIDE_FN - 1:
                        a_read(i, 1, st)
                else:
                    if x == 88 + WIDE_FN - 1:
                        # one row into k-step 1: every read of this stage has landed, every load of the next tile too
                        tr.need_all(out)
                        out += ["s_waitcnt vmcnt(0)", "s_barrier"]
                        a_read(0, 0, st ^ 1)
                    elif j == WIDE_FN - 1 and i > 0:
                        a_read(i, 0, st ^ 1)
                    if x >= 101 and (x - 101) % 3 == 0 and (x - 101) // 3 < WIDE_FN:
                        b_read(0, (x - 101) // 3, 0, st ^ 1)
                x += 1
    assert x == 176
    out += ["s_add_u32 %[ka], %[ka], 128", "s_add_u32 %[kb], %[kb], %[sb]"]
    return out


def wide_loop():
    out = []
    for w in range(4):
        out.append(f"s_mov_b32 s{80 + w}, %[da{w}]")
        out.append(f"s_mov_b32 s{84 + w}, %[db{w}]")
    tr = ReadTracker()
    # k-step 0 of tile 0: every A block and B set 0
    dummy = []
    for j in range(WIDE_FN):
        q = j & 1
        tr.read(out, ("b", 0, j), f"ds_read_b128 {wide_fb(0, j)}, %[lb0{q}] offset:{j * 4096}")
    for i in range(WIDE_FM):
        tr.read(out, ("a", i), f"ds_read_b128 {wide_fa(i)}, %[la0{i & 3}] offset:{i * 2048}")
    # The waits of a tile depend on the reads the tile before it left in flight.  Tile 0 follows the reads above; a
    # tile that follows another tile sees that tile's reads.  The waits written for the first case are the stricter
    # ones for the A blocks (their reads lie closer) - both cases are generated and compared, and the loop body uses
    # per-case text: the first trip's tiles are peeled.
    first0 = wide_k_tile(0, tr)
    first1 = wide_k_tile(1, tr)
    steady0 = wide_k_tile(0, tr)
    steady1 = wide_k_tile(1, tr)
    again0 = wide_k_tile(0, tr)
    assert again0 == steady0, "the schedule has not reached its steady state"
    # walk: tile 0 (first0); tile 1 (first1) if any; then pairs (steady0, steady1); then one more steady0 if odd
    out += ["s_cmp_lt_u32 %[n], 2", "s_cbranch_scc1 4f"]
    out += first0
    out += first1
    out += ["s_sub_u32 %[n], %[n], 2"]
    out.append("1:")
    out += ["s_cmp_lt_u32 %[n], 2", "s_cbranch_scc1 2f"]
    out += steady0
    out += steady1
    out += ["s_sub_u32 %[n], %[n], 2", "s_branch 1b", "2:"]
    out += ["s_cmp_eq_u32 %[n], 0", "s_cbranch_scc1 3f"]
    out += steady0
    out += ["s_branch 3f"]
    out.append("4:")   # a single tile
    out += first0
    out.append("3:")
    out += ["s_waitcnt vmcnt(0) lgkmcnt(0)", "s_nop 15", "s_nop 15"]
    return out


# ---- the 128 x 128 tile with four LDS stages: one workgroup per compute unit, loads three K tiles ahead -----------
# A wavefront owns 64 x 64 = 4 x 4 accumulator quads; a stage is 128 rows of A and 128 of B, 128 bytes each = 32 KiB,
# four of them a ring.  With at most one such workgroup on a compute unit (256 tiles or fewer) nothing else hides the
# latency of its loads: the two-stage loop of tile_gemm_kernel waits out every tile's loads there (0.67 us per K tile
# of 0.25 us of matrix instructions).  K tile t lies in stage t % 4:
#   k-step 0   multiplies fragment set 0, reads k-step 1 (same stage) into set 1
#   wait for the loads of tile t + 1 (at most those of tile t + 2 still in flight), barrier: every wavefront has read
#   stage (t - 1) % 4 for the last time and tile t + 1 has landed
#   k-step 1   multiplies set 1, reads tile t + 1's k-step 0 into set 0, issues the eight loads of tile t + 3 into
#              stage (t + 3) % 4
# B either K-contiguous (swizzled rows of 128 bytes, like A) or as it lies in memory ([k][n]: 64 k rows of 256 bytes,
# swizzled, read by ds_read_b64_tr_b16; one per-lane load offset and a scalar offset per load, as in the 256x256 loop).
# Fragment registers: set s, A block i at v[128 + 32 s + 4 i ..], B block j at v[144 + 32 s + 4 j ..].  LDS addresses:
# stages 0 / 1 and 2 / 3 share base registers (la{pair}{q}); the odd stage of a pair lies 32 KiB up, in the offset.
DEEP_STAGE = 32768
DEEP_B = 16384


def deep_fa(s, i):
    r = 128 + 32 * s + 4 * i
    return f"v[{r}:{r + 3}]"


def deep_fb(s, j):
    r = 144 + 32 * s + 4 * j
    return f"v[{r}:{r + 3}]"


def deep_fb_half(s, j, h):
    r = 144 + 32 * s + 4 * j + 2 * h
    return f"v[{r}:{r + 1}]"


DEEP_PITCH_TR = 256   # bytes between the k rows of a B tile kept as it lies in memory ([k][n], 128 columns)


def deep_reads(st, ks, to_set, tr):
    out = []
    pair, odd = st >> 1, st & 1
    order = [("a", 0)] + [("b", j) for j in range(4)] + [("a", i) for i in range(1, 4)]
    for kind, f in order:
        q = (2 * ks ^ f) & 3
        if kind == "a":
            out.append(f"ds_read_b128 {deep_fa(to_set, f)}, %[la{pair}{q}] offset:{odd * DEEP_STAGE + f * 2048}")
        elif tr == "pk":
            # B prepacked and kept in its pack order: block j lies in the wavefront's panel j / 2 (4 KiB a K tile),
            # rows 16 (j % 2) .. + 15; the matrix k-step reads the pack's k-steps 2 ks and 2 ks + 1 (1 KiB each); the
            # lane's chunk and row are in the one base register
            out.append(f"ds_read_b128 {deep_fb(to_set, f)}, %[lb{pair}0] offset:{odd * DEEP_STAGE + (f >> 1) * 4096 + ks * 2048 + (f & 1) * 256}")
        elif tr:
            # B as [k][n]: column block j in base j / 2, 32 bytes on for the odd one; the two reads give k 0-3 and 4-7
            # of the lane's chunk
            off = odd * DEEP_STAGE + (f & 1) * 32 + ks * 32 * DEEP_PITCH_TR
            out.append(f"ds_read_b64_tr_b16 {deep_fb_half(to_set, f, 0)}, %[lb{pair}{f >> 1}] offset:{off}")
            out.append(f"ds_read_b64_tr_b16 {deep_fb_half(to_set, f, 1)}, %[lb{pair}{f >> 1}] offset:{off + 4 * DEEP_PITCH_TR}")
        else:
            out.append(f"ds_read_b128 {deep_fb(to_set, f)}, %[lb{pair}{q}] offset:{odd * DEEP_STAGE + f * 2048}")
    return out


def deep_k_tile(st, tr):
    out = ["s_cmp_gt_i32 %[left], 0",
           "s_cselect_b32 s82, 0x7fffffff, 0",
           "s_cselect_b32 s86, 0x7fffffff, 0",
           "s_sub_u32 %[left], %[left], 1"]

    def mfma(x, s):
        i, j = x // 4, x % 4
        c = i * 4 + j
        return f"MFMA %[c{c}], {deep_fb(s, j)}, {deep_fa(s, i)}, %[c{c}]"
    reads = deep_reads(st, 1, 1, tr)
    out.append("s_waitcnt lgkmcnt(0)")
    for x in range(16):
        out.append(mfma(x, 0))
        if x < len(reads):
            out.append(reads[x])
    out += ["s_waitcnt vmcnt(8) lgkmcnt(0)", "s_barrier"]
    reads = deep_reads((st + 1) & 3, 0, 0, tr)
    target = (st + 3) & 3
    loads = []
    for p in range(4):
        loads.append(([f"s_add_u32 m0, %[m0w], {target * DEEP_STAGE + p * 4096}"],
                      f"buffer_load_dwordx4 %[ra{p}], s[80:83], %[ka] offen lds"))
    for p in range(4):
        m0 = f"s_add_u32 m0, %[m0w], {target * DEEP_STAGE + DEEP_B + p * 4096}"
        if tr is True:
            pre = [m0, "s_mov_b32 s88, %[kb]"] if p == 0 else [m0, "s_add_u32 s88, s88, %[pb]"]
            loads.append((pre, "buffer_load_dwordx4 %[rb0], s[84:87], s88 offen lds"))
        else:
            loads.append(([m0], f"buffer_load_dwordx4 %[rb{p}], s[84:87], %[kb] offen lds"))
    for x in range(16):
        if x % 2 == 0:
            out += loads[x // 2][0]
        out.append(mfma(x, 1))
        if x % 2 == 0:
            out.append(loads[x // 2][1])
        if 1 <= x <= len(reads):
            out.append(reads[x - 1])
    out += ["s_add_u32 %[ka], %[ka], 128", "s_add_u32 %[kb], %[kb], %[sb]"]
    return out


def deep_loop(tr):
    out = []
    for w in range(4):
        out.append(f"s_mov_b32 s{80 + w}, %[da{w}]")
        out.append(f"s_mov_b32 s{84 + w}, %[db{w}]")
    out += deep_reads(0, 0, 0, tr)
    out.append("1:")
    out += ["s_cmp_lt_u32 %[n], 4", "s_cbranch_scc1 2f"]
    for st in range(4):
        out += deep_k_tile(st, tr)
    out += ["s_sub_u32 %[n], %[n], 4", "s_branch 1b", "2:"]
    for st in range(3):
        out += [f"s_cmp_eq_u32 %[n], {st}", "s_cbranch_scc1 3f"]
        out += deep_k_tile(st, tr)
    out.append("3:")
    out += ["s_waitcnt vmcnt(0) lgkmcnt(0)", "s_nop 15", "s_nop 15"]
    return out


def as_macro(name, lines):
    text = f"#define {name}(MFMA) \\\n"
    body = []
    for line in lines:
        if line.startswith("MFMA "):
            body.append('  MFMA "' + line[4:] + '\\n\\t"')
        else:
            body.append('  "' + line + '\\n\\t"')
    return text + " \\\n".join(body) + "\n"


def main():
    w = sys.stdout.write
    w("// Generated by gen_tile_loop.py (python3 gen_tile_loop.py > tile_loop_asm.inc): the K loop of the 256x256 tile\n")
    w("// on the 16x16 matrix instructions.  VECOPS_LOOP256_K: both operands K-contiguous in LDS; VECOPS_LOOP256_TR: B as\n")
    w("// it lies in memory ([k][n]) and transposed by the LDS reads.  MFMA: the instruction's mnemonic, a string.\n")
    w(as_macro("VECOPS_LOOP256_K", loop(False)))
    w("\n")
    w(as_macro("VECOPS_LOOP256_TR", loop(True)))
    w("\n// VECOPS_LOOP256_PK: B prepacked (vecops_hip_pack_b) and kept in its pack order in LDS.\n")
    w(as_macro("VECOPS_LOOP256_PK", loop("pk")))
    w("\n// The K loop of the 256 x 352 tile (8-bit operands, both K-contiguous): see gen_tile_loop.py.\n")
    w(as_macro("VECOPS_LOOP352_K", wide_loop()))
    w("\n// its 88 accumulator quads: 64 in accumulation registers, 24 in vector registers\n")
    w("#define VECOPS_LOOP352_ACCUMULATORS(t) \\\n  " +
      ", \\\n  ".join(", ".join(f'[c{x}] "+{"a" if x < 64 else "v"}"(t[{x}])' for x in range(r, r + 4)) for r in range(0, 88, 4)) + "\n")
    w("#define VECOPS_LOOP352_CLOBBERS \\\n  " + ", ".join(f'"s{r}"' for r in range(80, 89)) + ", \\\n  " +
      ", \\\n  ".join(", ".join(f'"v{r}"' for r in range(b, min(b + 16, 248))) for b in range(128, 248, 16)) + "\n")
    w("\n// The K loop of the 128 x 128 tile on four LDS stages (one workgroup per compute unit): see gen_tile_loop.py.\n")
    w(as_macro("VECOPS_LOOP128_DEEP", deep_loop(False)))
    w("\n// ... with B as it lies in memory ([k][n]), transposed by the LDS reads\n")
    w(as_macro("VECOPS_LOOP128_DEEP_TR", deep_loop(True)))
    w("\n// The same with B prepacked (vecops_hip_pack_b's layout, kept in its own order in LDS).\n")
    w(as_macro("VECOPS_LOOP128_DEEP_PK", deep_loop("pk")))
    w("#define VECOPS_LOOP128_ACCUMULATORS(t) \\\n  " +
      ", \\\n  ".join(", ".join(f'[c{x}] "+a"(t[{x // 4}][{x % 4}])' for x in range(r, r + 4)) for r in range(0, 16, 4)) + "\n")
    w("#define VECOPS_LOOP128_CLOBBERS \\\n  " + ", ".join(f'"s{r}"' for r in range(80, 89)) + ", \\\n  " +
      ", \\\n  ".join(", ".join(f'"v{r}"' for r in range(b, b + 16)) for b in range(128, 192, 16)) + "\n")
    w("\n// the accumulators as operands: quad x = t[x / 8][x % 8]\n")
    w("#define VECOPS_LOOP256_ACCUMULATORS(t) \\\n  " +
      ", \\\n  ".join(", ".join(f'[c{x}] "+a"(t[{x // 8}][{x % 8}])' for x in range(r, r + 4)) for r in range(0, 64, 4)) + "\n")
    w("\n// registers the loop uses by number\n")
    w("#define VECOPS_LOOP256_CLOBBERS \\\n  " + ", ".join(f'"s{r}"' for r in range(80, 89)) + ", \\\n  " +
      ", \\\n  ".join(", ".join(f'"v{r}"' for r in range(b, b + 16)) for b in range(128, 256, 16)) + "\n")


if __name__ == "__main__":
    main()
