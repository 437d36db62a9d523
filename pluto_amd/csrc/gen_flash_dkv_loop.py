#!/usr/bin/env python3
"""Writes flash_dkv_loop.inc: the hand-scheduled gfx950 instruction stream of
the key-owned attention backward kernel for heads of 64 channels
(flash_dkv_wide.hip), the body of one `asm volatile` statement with a fixed
register allocation.

A wave owns 64 keys (two halves c of 32, lane = key) and walks the query blocks
of 32 rows that see them.  Per block and half:

  S  = Q K^T - lse / scale,  dP = dO V^T - delta     8 matrix instructions
  P  = 2^(S scale log2 e),   dS = P dP               64 vector instructions
  dV^T += dO^T P,            dK^T += Q^T dS          8 matrix instructions

K and V stay in registers as B operands, so every A operand read from LDS (rows
of Q and dO for the first pair of products, their transposes for the second)
feeds two matrix instructions, one per half: half of the LDS traffic per matrix
instruction of a 32-key wave, which is what keeps four waves a compute unit
below the LDS bandwidth.  With 128 accumulator registers, 64 operand registers
for K and V (all in AGPRs) and the pipeline's buffers a wave uses 448 of the 512
registers of a SIMD lane: one wave a SIMD, so nothing but the order of its own
instructions keeps the matrix pipe busy.  The order, per block b, two slots:

  slot 1   matrix: dV, dK (block b-1, half 0); S, dP (block b, half 0)
           vector: P, dS of (block b-1, half 1)
           LDS:    row statistics and Q / dO rows of block b
  slot 2   matrix: dV, dK (block b-1, half 1); S, dP (block b, half 1)
           vector: P, dS of (block b, half 0)
           LDS:    transposed Q / dO operands of block b

Every matrix instruction is followed by four vector instructions and at most
two LDS reads, none of which waits for a result of the same slot.

Query blocks travel global -> LDS (Q rows, dO rows, 32 + 32 row statistics) through a
ring of eight stages; one workgroup barrier per block hands a stage over, and a
block is requested six barriers before its rows are read.  The two waves of a
workgroup share the stream; the second wave's keys start 64 rows later, so it
idles (barrier and requests only) for the first two blocks.

A wave's first three blocks (the causal diagonal crosses them) and its last one
(the sequence may end inside it) run a variant of the slots that compares every
element's query row with two per-lane bounds.

Usage: python gen_flash_dkv_loop.py [output]   (default: flash_dkv_loop.inc
beside this file)
"""
import os
import sys

D = 64
KS = D // 16            # contraction steps of the row products
DB = D // 32            # 32-channel blocks of dK^T, dV^T
RING = 8                # LDS stages
TILE_BYTES = 32 * D * 2
STAT_BYTES = 256
STAGE_BYTES = 2 * TILE_BYTES + 2 * STAT_BYTES
ROW_BYTES = D * 2
FILL_OPS = 5            # vector-memory operations a wave and stage: 2 Q, 2 dO, 1 statistics


class Registers:
    def __init__(self):
        # v128..v255 carry dK, dV out of the statement; until then they hold the pipeline
        self.SB = [(128, 144), (160, 176)]            # [c] -> (S, dP), 16 registers each
        self.PB = [([192, 196], [200, 204]),          # [c] -> (P[s2], dS[s2]), 4 registers each
                   ([208, 212], [216, 220])]
        self.ROWQ = [224 + 4 * ks for ks in range(KS)]
        self.ROWG = [240 + 4 * ks for ks in range(KS)]
        self.OUT_DK = [[128, 144], [160, 176]]        # [c][db]
        self.OUT_DV = [[192, 208], [224, 240]]
        # v64..v127 bring K and V in; then transposed operands and row statistics
        self.KIN = [[64 + 16 * c + 4 * ks for ks in range(KS)] for c in range(2)]
        self.VIN = [[96 + 16 * c + 4 * ks for ks in range(KS)] for c in range(2)]
        self.TRG = [[64 + 8 * s2 + 4 * db for db in range(DB)] for s2 in range(2)]
        self.TRQ = [[80 + 8 * s2 + 4 * db for db in range(DB)] for s2 in range(2)]
        self.LSE = 96
        self.DEL = 112
        # inputs
        at = 32
        def take(n=1):
            nonlocal at
            first = at
            at += n
            return first
        self.ROWADDR = [take() for _ in range(KS)]
        self.TRADDR = [take() for _ in range(DB)]
        self.STATADDR = take()
        self.QFILL = [take(), take()]
        self.GFILL = [take(), take()]
        self.SFILL = take()
        self.N4 = take()
        self.TL4 = take()
        self.inputs_end = at
        # temporaries
        self.ROWDYN = [take() for _ in range(KS)]
        self.TRDYN = [take() for _ in range(DB)]
        self.STATDYN = take()
        self.FTMP = [take() for _ in range(FILL_OPS)]
        self.F = take()
        self.LIM = take()
        self.NEG = take()
        self.temps_end = at
        assert at <= 64
        # AGPRs
        self.DK = [[16 * (2 * c + db) for db in range(DB)] for c in range(2)]
        self.DV = [[64 + 16 * (2 * c + db) for db in range(DB)] for c in range(2)]
        self.KF = [[128 + 4 * (KS * c + ks) for ks in range(KS)] for c in range(2)]
        self.VF = [[160 + 4 * (KS * c + ks) for ks in range(KS)] for c in range(2)]
        self.agprs = 192


def vt(base, n):
    return "v[%d:%d]" % (base, base + n - 1) if n > 1 else "v%d" % base


def at_(base, n):
    return "a[%d:%d]" % (base, base + n - 1) if n > 1 else "a%d" % base


MFMA = "v_mfma_f32_32x32x16_bf16"


class Emitter:
    def __init__(self):
        self.r = Registers()
        self.lines = []
        self.label_count = 0
        self.lds_queue = []

    def emit(self, text):
        self.lines.append(text)

    # ---- LDS reads with lgkmcnt bookkeeping (reads return in order, the counter holds 15) ----
    def lds_read(self, text, dest):
        if len(self.lds_queue) >= 15:
            self.emit("s_waitcnt lgkmcnt(14)")
            self.lds_queue = self.lds_queue[len(self.lds_queue) - 14:]
        self.emit(text)
        self.lds_queue.append(dest)

    def wait_for(self, dest):
        """dest: a destination, or a kind ("trg", "row" ...) for all of that kind."""
        last = -1
        for i, d in enumerate(self.lds_queue):
            if d == dest or (isinstance(d, tuple) and d[0] == dest):
                last = i
        if last < 0:
            return
        younger = len(self.lds_queue) - 1 - last
        self.emit("s_waitcnt lgkmcnt(%d)" % younger)
        self.lds_queue = self.lds_queue[last + 1:]

    # ---- reads of one block ------------------------------------------------------------------
    def stat_reads(self):
        """Eight reads: register i of LSE / DEL <- statistic of query 8 (i / 4) + 4 h + i % 4."""
        r = self.r
        out = []
        for name, base, offset in (("lse", r.LSE, 0), ("del", r.DEL, STAT_BYTES)):
            for j in range(4):
                out.append(("ds_read_b128 %s, v%d offset:%d" %
                            (vt(base + 4 * j, 4), r.STATDYN, offset + 32 * j), name))
        return out

    def row_reads(self):
        r = self.r
        out = []
        for ks in range(KS):
            out.append(("ds_read_b128 %s, v%d" % (vt(r.ROWQ[ks], 4), r.ROWDYN[ks]), ("row", "q", ks)))
            out.append(("ds_read_b128 %s, v%d offset:%d" %
                        (vt(r.ROWG[ks], 4), r.ROWDYN[ks], TILE_BYTES), ("row", "g", ks)))
        return out

    def first_half_reads(self):
        """Statistics and rows in the order the first products need them."""
        stats = self.stat_reads()
        rows = self.row_reads()
        lse, dele = stats[:4], stats[4:]
        return lse + rows[0:1] + dele + rows[1:]

    def transposed_reads(self):
        r = self.r
        out = []
        for name, regs, tile in (("trg", r.TRG, TILE_BYTES), ("trq", r.TRQ, 0)):
            for s2 in range(2):
                for db in range(DB):
                    for part in range(2):
                        out.append(("ds_read_b64_tr_b16 %s, v%d offset:%d" %
                                    (vt(regs[s2][db] + 2 * part, 2), r.TRDYN[db],
                                     tile + (16 * s2 + 8 * part) * ROW_BYTES), (name, s2, db)))
        return out

    # ---- vector side of one (block, half) ---------------------------------------------------------
    def vector_items(self, c, masked):
        r = self.r
        S, DP = r.SB[c]
        P, DS = r.PB[c]
        items = []
        for e in range(8):
            a, b = 2 * e, 2 * e + 1
            if masked:
                for i in (a, b):
                    ci = 8 * (i // 4) + i % 4
                    items.append("v_cmp_lt_i32 vcc, %d, v%d" % (ci, r.F))
                    items.append("v_cmp_gt_i32_e64 %%[mpair], %d, v%d" % (ci, r.LIM))
                    items.append("s_or_b64 vcc, vcc, %[mpair]")
                    items.append("v_cndmask_b32 v%d, v%d, v%d, vcc" % (S + i, S + i, r.NEG))
            items.append("v_mul_f32 v%d, %%[scale2], v%d" % (S + a, S + a))
            items.append("v_mul_f32 v%d, %%[scale2], v%d" % (S + b, S + b))
            items.append("v_exp_f32 v%d, v%d" % (S + a, S + a))
            items.append("v_exp_f32 v%d, v%d" % (S + b, S + b))
            items.append("v_mul_f32 v%d, v%d, v%d" % (DP + a, S + a, DP + a))
            items.append("v_mul_f32 v%d, v%d, v%d" % (DP + b, S + b, DP + b))
            s2, w = divmod(e, 4)
            items.append("v_cvt_pk_bf16_f32 v%d, v%d, v%d" % (P[s2] + w, S + a, S + b))
            items.append("v_cvt_pk_bf16_f32 v%d, v%d, v%d" % (DS[s2] + w, DP + a, DP + b))
        return items

    def mask_bounds(self, plus_f, plus_lim):
        """F and LIM for the block whose first query is 32 * bcount - plus... rows
        from the wave's first key: hidden where ci < F or ci > LIM."""
        r = self.r
        e = self.emit
        e("s_lshl_b32 %[t0], %[bcount], 5")
        if plus_f:
            e("s_sub_u32 %%[t1], %%[t0], %d" % plus_f)
            e("v_subrev_u32 v%d, %%[t1], v%d" % (r.F, r.N4))
        else:
            e("v_subrev_u32 v%d, %%[t0], v%d" % (r.F, r.N4))
        if plus_lim:
            e("s_sub_u32 %%[t1], %%[t0], %d" % plus_lim)
            e("v_subrev_u32 v%d, %%[t1], v%d" % (r.LIM, r.TL4))
        else:
            e("v_subrev_u32 v%d, %%[t0], v%d" % (r.LIM, r.TL4))

    # ---- matrix side ------------------------------------------------------------------------------
    def accumulate_products(self, c):
        """dV^T, dK^T of half c from the transposed operands and PB[c]: 8 instructions."""
        r = self.r
        P, DS = r.PB[c]
        out = []
        for s2 in range(2):
            for db in range(DB):
                acc = at_(r.DV[c][db], 16)
                out.append(("trg" if (s2, db) == (0, 0) else None, "%s %s, %s, %s, %s" %
                            (MFMA, acc, vt(r.TRG[s2][db], 4), vt(P[s2], 4), acc)))
        for s2 in range(2):
            for db in range(DB):
                acc = at_(r.DK[c][db], 16)
                out.append(("trq" if (s2, db) == (0, 0) else None, "%s %s, %s, %s, %s" %
                            (MFMA, acc, vt(r.TRQ[s2][db], 4), vt(DS[s2], 4), acc)))
        return out

    def score_products(self, c):
        """S, dP of half c from the row operands: 8 instructions, the two chains alternating."""
        r = self.r
        S, DP = r.SB[c]
        out = []
        for ks in range(KS):
            acc = vt(S, 16)
            out.append(({0: [("row", "q", 0), "lse"], 1: ["row"]}.get(ks, []),
                        "%s %s, %s, %s, %s" % (MFMA, acc, vt(r.ROWQ[ks], 4), at_(r.KF[c][ks], 4),
                                               vt(r.LSE, 16) if ks == 0 else acc)))
            acc = vt(DP, 16)
            out.append(({0: [("row", "g", 0), "del"]}.get(ks, []),
                        "%s %s, %s, %s, %s" % (MFMA, acc, vt(r.ROWG[ks], 4), at_(r.VF[c][ks], 4),
                                               vt(r.DEL, 16) if ks == 0 else acc)))
        return out

    # ---- one slot ---------------------------------------------------------------------------------
    def slot(self, c, accumulate, scores, vector, masked, reads, reads_from=0, reads_per_gap=2):
        """Matrix instructions of half c, the vector items of the other buffer,
        `reads` (text, destination) spread `reads_per_gap` a gap from gap `reads_from` on."""
        matrix = []
        if accumulate:
            matrix += [([need] if need else [], text) for need, text in self.accumulate_products(c)]
        if scores:
            matrix += self.score_products(c)
        items = []
        if vector:
            items += self.vector_items(1 - c, masked)
        gaps = max(len(matrix), 1)
        # the last gap stays free of vector work: the next slot's first matrix
        # instruction reads what this slot's last conversions write
        per_gap = (len(items) + max(gaps - 2, 0)) // max(gaps - 1, 1) if gaps > 1 else len(items)
        reads = list(reads)
        at = 0
        for g in range(gaps):
            if matrix:
                needs, text = matrix[g]
                for need in needs:
                    self.wait_for(need)
                self.emit(text)
            if g >= reads_from:
                for text, dest in reads[:reads_per_gap]:
                    self.lds_read(text, dest)
                reads = reads[reads_per_gap:]
            for text in items[at:at + per_gap]:
                self.emit(text)
            at += per_gap
        for text, dest in reads:
            self.lds_read(text, dest)
        for text in items[at:]:
            self.emit(text)

    # ---- barrier, hand-over of a stage, request of the block six ahead --------------------------------
    def fill_from(self, stage_scalar=None, stage=None):
        """Requests the block at the running offsets into a stage.  The offsets are
        added into the lanes' (a descriptor's range check sees the vector offset
        only); the updates of the running offsets sit between a write of M0 and
        the request that reads it (one wait state)."""
        r = self.r
        e = self.emit
        e("v_add_u32 v%d, %%[qoff], v%d" % (r.FTMP[0], r.QFILL[0]))
        e("v_add_u32 v%d, %%[qoff], v%d" % (r.FTMP[1], r.QFILL[1]))
        e("v_add_u32 v%d, %%[goff], v%d" % (r.FTMP[2], r.GFILL[0]))
        e("v_add_u32 v%d, %%[goff], v%d" % (r.FTMP[3], r.GFILL[1]))
        e("v_add_u32 v%d, %%[soff], v%d" % (r.FTMP[4], r.SFILL))
        if stage_scalar is None:
            e("s_add_u32 m0, %%[ldsq], %d" % (stage * STAGE_BYTES))
        else:
            e("s_add_u32 m0, %%[ldsq], %s" % stage_scalar)
        e("s_add_u32 %%[soff], %%[soff], %d" % 128)
        e("buffer_load_dwordx4 v%d, %%[qrsrc], 0 offen lds" % r.FTMP[0])
        e("buffer_load_dwordx4 v%d, %%[qrsrc], 0 offen offset:1024 lds" % r.FTMP[1])
        if stage_scalar is None:
            e("s_add_u32 m0, %%[ldsq], %d" % (stage * STAGE_BYTES + TILE_BYTES))
        else:
            e("s_add_u32 m0, m0, %d" % TILE_BYTES)
        e("s_add_u32 %[qoff], %[qoff], %[qstep]")
        e("buffer_load_dwordx4 v%d, %%[grsrc], 0 offen lds" % r.FTMP[2])
        e("buffer_load_dwordx4 v%d, %%[grsrc], 0 offen offset:1024 lds" % r.FTMP[3])
        if stage_scalar is None:
            e("s_add_u32 m0, %%[ldss], %d" % (stage * STAGE_BYTES))
        else:
            e("s_add_u32 m0, %%[ldss], %s" % stage_scalar)
        e("s_add_u32 %[goff], %[goff], %[gstep]")
        e("buffer_load_dword v%d, %%[srsrc], 0 offen lds" % r.FTMP[4])

    def step_barrier(self):
        """Starts step s = tcount: block s has landed for every wave, everyone is
        done with block s - 2, whose stage takes block s + RING - 2."""
        e = self.emit
        e("s_waitcnt vmcnt(%d)" % (FILL_OPS * (RING - 3)))
        e("s_barrier")
        e("s_add_u32 %%[t0], %%[tcount], %d" % (RING - 2))
        e("s_and_b32 %%[t0], %%[t0], %d" % (RING - 1))
        e("s_mul_i32 %%[t0], %%[t0], %d" % STAGE_BYTES)
        self.fill_from(stage_scalar="%[t0]")
        e("s_add_u32 %[tcount], %[tcount], 1")

    def block_addresses(self):
        """LDS addresses of the block of the step just started (tcount - 1)."""
        r = self.r
        e = self.emit
        e("s_sub_u32 %[t0], %[tcount], 1")
        e("s_and_b32 %%[t0], %%[t0], %d" % (RING - 1))
        e("s_mul_i32 %%[t0], %%[t0], %d" % STAGE_BYTES)
        e("s_add_u32 %[t0], %[t0], %[ldsbase]")
        out = []
        for ks in range(KS):
            out.append("v_add_u32 v%d, %%[t0], v%d" % (r.ROWDYN[ks], r.ROWADDR[ks]))
        out.append("v_add_u32 v%d, %%[t0], v%d" % (r.STATDYN, r.STATADDR))
        for db in range(DB):
            out.append("v_add_u32 v%d, %%[t0], v%d" % (r.TRDYN[db], r.TRADDR[db]))
        return out

    # ---- iterations ---------------------------------------------------------------------------------
    def iteration(self, masked):
        """Block b = bcount, 1 <= b < n."""
        self.step_barrier()
        for text in self.block_addresses():
            self.emit(text)
        if masked:
            self.mask_bounds(64, 32)      # (block b-1, half 1)
        self.wait_for("trq")
        self.slot(0, True, True, True, masked, self.first_half_reads(), reads_from=0, reads_per_gap=4)
        if masked:
            self.mask_bounds(0, 0)        # (block b, half 0)
        self.slot(1, True, True, True, masked, self.transposed_reads(), reads_from=8, reads_per_gap=4)

    def first_iteration(self):
        """Block 0: no products owed yet."""
        e = self.emit
        self.step_barrier()
        for text in self.block_addresses():
            e(text)
        for text, dest in self.first_half_reads():
            self.lds_read(text, dest)
        self.slot(0, False, True, False, False, [])
        self.mask_bounds(0, 0)
        self.slot(1, False, True, True, True, self.transposed_reads(), reads_per_gap=4)

    def drain(self):
        """Step n: the products of block n - 1."""
        e = self.emit
        self.step_barrier()
        self.mask_bounds(64, 32)
        self.slot(0, True, False, True, True, [])
        e("s_nop 7")
        self.slot(1, True, False, False, False, [])

    def build(self):
        r = self.r
        e = self.emit
        e("s_mov_b32 %[m0save], m0")
        e("s_waitcnt lgkmcnt(0)")
        # the first blocks are requested while K and V are still on their way
        for stage in range(RING - 2):
            self.fill_from(stage=stage)
        e("s_waitcnt vmcnt(%d)" % (FILL_OPS * (RING - 2)))
        # K, V operands to AGPRs; accumulators to zero
        for c in range(2):
            for ks in range(KS):
                for i in range(4):
                    e("v_accvgpr_write_b32 a%d, v%d" % (r.KF[c][ks] + i, r.KIN[c][ks] + i))
                    e("v_accvgpr_write_b32 a%d, v%d" % (r.VF[c][ks] + i, r.VIN[c][ks] + i))
        for i in range(128):
            e("v_accvgpr_write_b32 a%d, 0" % i)
        e("v_mov_b32 v%d, 0xf149f2ca" % r.NEG)      # -1e30: 2^(that * scale) is zero
        idle, start, top, masked, drain, finish = ("Lidle_%=", "Lstart_%=", "Ltop_%=", "Lmasked_%=",
                                                   "Ldrain_%=", "Lfinish_%=")
        e("%s:" % idle)
        e("s_cmp_eq_u32 %[idle], 0")
        e("s_cbranch_scc1 %s" % start)
        self.step_barrier()
        e("s_sub_u32 %[idle], %[idle], 1")
        e("s_branch %s" % idle)
        e("%s:" % start)
        e("s_cmp_eq_u32 %[nblk], 0")
        e("s_cbranch_scc1 %s" % finish)
        e("s_mov_b32 %[bcount], 0")
        self.first_iteration()
        e("s_mov_b32 %[bcount], 1")
        at_top = list(self.lds_queue)
        e("%s:" % top)
        e("s_cmp_eq_u32 %[bcount], %[nblk]")
        e("s_cbranch_scc1 %s" % drain)
        e("s_cmp_le_u32 %[bcount], 2")
        e("s_cbranch_scc1 %s" % masked)
        e("s_add_u32 %[t0], %[bcount], 1")
        e("s_cmp_eq_u32 %[t0], %[nblk]")
        e("s_cbranch_scc1 %s" % masked)
        self.iteration(False)
        assert self.lds_queue == at_top, (self.lds_queue, at_top)
        e("s_add_u32 %[bcount], %[bcount], 1")
        e("s_branch %s" % top)
        e("%s:" % masked)
        self.lds_queue = list(at_top)
        self.iteration(True)
        assert self.lds_queue == at_top
        e("s_add_u32 %[bcount], %[bcount], 1")
        e("s_branch %s" % top)
        e("%s:" % drain)
        self.lds_queue = list(at_top)
        self.drain()
        e("%s:" % finish)
        # requests beyond the last block are still on their way into LDS
        e("s_waitcnt vmcnt(0) lgkmcnt(0)")
        e("s_nop 15")
        e("s_nop 15")
        e("s_barrier")
        for c in range(2):
            for db in range(DB):
                for i in range(16):
                    e("v_accvgpr_read_b32 v%d, a%d" % (r.OUT_DK[c][db] + i, r.DK[c][db] + i))
                    e("v_accvgpr_read_b32 v%d, a%d" % (r.OUT_DV[c][db] + i, r.DV[c][db] + i))
        e("s_mov_b32 m0, %[m0save]")


def c_string(lines, indent="  "):
    return "\n".join('%s"%s\\n\\t"' % (indent, line.replace("\n", "\\n").replace("\t", "\\t"))
                     for line in lines)


def render():
    g = Emitter()
    g.build()
    r = g.r
    name = "FLASH_DKV_D64"
    out = ["// heads of 64 channels, two waves a workgroup: %d instructions and labels" % len(g.lines)]
    out.append("#define %s_ASM \\" % name)
    out.append(" \\\n".join(c_string(g.lines).split("\n")))
    out.append("")

    def define(tag, value):
        out.append("#define %s_%s %s" % (name, tag, value))

    for c in range(2):
        for db in range(DB):
            define("DK%d%d" % (c, db), '"=&{%s}"' % vt(r.OUT_DK[c][db], 16))
            define("DV%d%d" % (c, db), '"=&{%s}"' % vt(r.OUT_DV[c][db], 16))
        for ks in range(KS):
            define("K%d%d" % (c, ks), '"+{%s}"' % vt(r.KIN[c][ks], 4))
            define("V%d%d" % (c, ks), '"+{%s}"' % vt(r.VIN[c][ks], 4))
    for ks in range(KS):
        define("ROWADDR%d" % ks, '"{v%d}"' % r.ROWADDR[ks])
    for db in range(DB):
        define("TRADDR%d" % db, '"{v%d}"' % r.TRADDR[db])
    define("STATADDR", '"{v%d}"' % r.STATADDR)
    for i in range(2):
        define("QFILL%d" % i, '"{v%d}"' % r.QFILL[i])
        define("GFILL%d" % i, '"{v%d}"' % r.GFILL[i])
    define("SFILL", '"{v%d}"' % r.SFILL)
    define("N4", '"{v%d}"' % r.N4)
    define("TL4", '"{v%d}"' % r.TL4)
    clobbers = ['"v%d"' % v for v in range(r.inputs_end, r.temps_end)]
    clobbers += ['"a%d"' % a for a in range(r.agprs)]
    define("CLOBBERS", ", ".join(clobbers) + ', "vcc", "scc", "memory"')
    define("RING", str(RING))
    define("STAGE_BYTES", str(STAGE_BYTES))
    define("TILE_BYTES", str(TILE_BYTES))
    return "\n".join(out) + "\n"


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    target = sys.argv[1] if len(sys.argv) > 1 else os.path.join(here, "flash_dkv_loop.inc")
    text = ("// Generated by gen_flash_dkv_loop.py; do not edit.  The instruction stream of the\n"
            "// main loop of flash_dkv_wide_kernel, see the generator for the schedule.\n\n")
    text += render()
    with open(target, "w") as f:
        f.write(text)


if __name__ == "__main__":
    main()
