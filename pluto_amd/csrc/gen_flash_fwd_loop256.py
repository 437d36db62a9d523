#!/usr/bin/env python3
"""Writes flash_fwd_loop256.inc: the hand-scheduled gfx950 instruction stream of
the causal flash-attention forward kernel's main loop at head width 256
(flash_fwd_pipelined.hip), the body of one `asm volatile` statement with a
fixed register allocation.

The schedule is the one of gen_flash_fwd_loop.py, per 32-key block b:

    matrix:  S^T(b+1) = K(b+1) Q^T                      16 instructions
             l, O^T  += [1; V^T(b-1)] P^T(b-1)           2 + 16 instructions
    vector:  softmax of block b
    LDS:     V^T operands of block b-1 into the registers the K operands of
             block b+1 have just left, K operands of block b+2 into the
             registers the V^T operands leave

What the width changes.  O^T is 8 x 16 registers a lane and Q^T 64: both live
in AGPRs (the matrix instructions read and write them there; the rare rescale
of O^T copies through vector registers), the pipeline in 200 vector registers:
448 of a SIMD lane's 512, one wave a SIMD, four waves (128 query rows) a
workgroup.  With 34 matrix instructions against the same softmax per block as
at the narrower widths, one wave's instruction stream keeps the matrix pipe
busy without a partner.  A block of K or V is 16 KiB, so the LDS ring holds
single blocks: unit t = {K(t+3), V(t)} in stage t mod 4 of 32 KiB.  Iteration b
reads K(b+2) and V(b-1) from the same unit b-1; the workgroup barrier that
starts the iteration hands unit b-2's stage to unit b+2, three iterations
before it is read.  Stage addresses are computed (one scalar, six vector adds
an iteration), so the loop is unrolled by the two block parities only.

Usage: python gen_flash_fwd_loop256.py [output]   (default: flash_fwd_loop256.inc
beside this file)
"""
import os
import sys

D = 256
WAVES = 4
KS = D // 16
DB = D // 32
ROW_BYTES = D * 2
BLOCK_BYTES = 32 * ROW_BYTES          # one block of K or of V
STAGE_BYTES = 2 * BLOCK_BYTES
STAGES = 4
LOADS = BLOCK_BYTES // (64 * WAVES * 16)   # 16-byte loads a lane, tensor and block
MFMA = "v_mfma_f32_32x32x16_bf16"


def vt(base, n):
    return "v[%d:%d]" % (base, base + n - 1) if n > 1 else "v%d" % base


def at(base, n):
    return "a[%d:%d]" % (base, base + n - 1) if n > 1 else "a%d" % base


class Registers:
    def __init__(self):
        # v128..v255: the pipeline, and O^T on the way out
        self.OUT = [128 + 16 * db for db in range(DB)]
        self.S = [128, 144]
        self.OP = [160 + 4 * j for j in range(KS)]
        self.PF = [[224, 228], [232, 236]]            # [parity][s2]
        self.RT = [240, 241, 242, 243]                # rescale copies
        self.QIN = self.OP                            # Q^T arrives where the operands will live
        low = 60

        def take(n=1, align=1):
            nonlocal low
            low += (-low) % align
            first = low
            low += n
            return first
        # inputs and in-outs
        self.KADDR = [take() for _ in range(4)]       # row reads: contraction steps ks % 4
        self.VADDR = [take() for _ in range(2)]       # transposing reads: channel blocks db % 2
        self.KFILL = [take() for _ in range(LOADS)]
        self.VFILL = [take() for _ in range(LOADS)]
        self.ROWLIM = take()
        self.MUSED = take()
        self.MTRUE = take()
        self.THR = take()
        self.ONES = take(4, 4)
        self.L = take(16, 4)
        self.pinned_end = low
        # temporaries
        self.KDYN = [take() for _ in range(4)]
        self.VDYN = [take() for _ in range(2)]
        self.FTMP = [take() for _ in range(2 * LOADS)]
        self.T0 = take()
        self.T1 = take()
        self.ALPHA = take()
        self.LIM = take()
        self.KMASK = take()
        self.temps_end = low
        assert low <= 128
        self.O = [16 * db for db in range(DB)]        # AGPRs
        self.QF = [128 + 4 * ks for ks in range(KS)]
        self.agprs = 192


class Emitter:
    def __init__(self):
        self.r = Registers()
        self.lines = []
        self.label_count = 0
        self.lds_queue = []

    def emit(self, text):
        self.lines.append(text)

    def label(self, stem):
        self.label_count += 1
        return "L%s_%d_%%=" % (stem, self.label_count)

    # ---- LDS reads with lgkmcnt bookkeeping (reads return in order; the counter holds 15) ----
    def lds_read(self, text, dest):
        if len(self.lds_queue) >= 15:
            self.emit("s_waitcnt lgkmcnt(14)")
            self.lds_queue = self.lds_queue[len(self.lds_queue) - 14:]
        self.emit(text)
        self.lds_queue.append(dest)

    def wait_for(self, dest):
        last = -1
        for i, d in enumerate(self.lds_queue):
            if d == dest:
                last = i
        if last < 0:
            return
        younger = len(self.lds_queue) - 1 - last
        self.emit("s_waitcnt lgkmcnt(%d)" % younger)
        self.lds_queue = self.lds_queue[last + 1:]

    def k_read(self, ks):
        """K operand tuple ks of the block in the stage KDYN points at."""
        r = self.r
        self.lds_read("ds_read_b128 %s, v%d offset:%d" %
                      (vt(r.OP[ks], 4), r.KDYN[ks % 4], 128 * (ks // 4)), ("op", ks))

    def v_read(self, j):
        """V^T operand tuple j = (s2, db) of the block in the stage VDYN points at."""
        r = self.r
        s2, db = divmod(j, DB)
        offset = BLOCK_BYTES + 128 * (db // 2) + 16 * s2 * ROW_BYTES
        base = r.VDYN[db % 2]
        self.lds_read("ds_read_b64_tr_b16 %s, v%d offset:%d" % (vt(r.OP[j], 2), base, offset),
                      ("op", j))
        self.lds_read("ds_read_b64_tr_b16 %s, v%d offset:%d" %
                      (vt(r.OP[j] + 2, 2), base, offset + 8 * ROW_BYTES), ("op", j))

    # ---- global -> LDS ----------------------------------------------------------------------------
    def request(self, stage=None, k_part=True, v_part=True, spread=False):
        """K rows at byte offset %[koff], V rows at %[voff] into a stage (a number,
        or the byte offset in %[t2]).  The running offsets are added into the
        lanes' (a descriptor's range check sees the vector offset only).  Returns
        the requests themselves when `spread` (the caller deals them out between
        its matrix instructions: four waves that issue eight requests each right
        after a barrier queue behind each other at the compute unit's one
        address path for 500 cycles), else emits them.  A write of M0 and the
        request that reads it are never adjacent."""
        r = self.r
        e = self.emit
        if k_part:
            for i in range(LOADS):
                e("v_add_u32 v%d, %%[koff], v%d" % (r.FTMP[i], r.KFILL[i]))
            e("s_add_u32 %[koff], %[koff], %[kstep]")
        if v_part:
            for i in range(LOADS):
                e("v_add_u32 v%d, %%[voff], v%d" % (r.FTMP[LOADS + i], r.VFILL[i]))
            e("s_add_u32 %[voff], %[voff], %[vstep]")
        out = []
        if k_part:
            if stage is None:
                out.append("s_add_u32 m0, %[ldsw], %[t2]")
            else:
                out.append("s_add_u32 m0, %%[ldsw], %d" % (stage * STAGE_BYTES))
            for i in range(LOADS):
                out.append("buffer_load_dwordx4 v%d, %%[krsrc], 0 offen%s lds" %
                           (r.FTMP[i], " offset:%d" % (1024 * i) if i else ""))
        if v_part:
            if stage is None:
                if k_part:
                    out.append("s_add_u32 m0, m0, %d" % BLOCK_BYTES)
                else:
                    out.append("s_add_u32 m0, %%[t2], %d\n\ts_add_u32 m0, m0, %%[ldsw]" % BLOCK_BYTES)
            else:
                out.append("s_add_u32 m0, %%[ldsw], %d" % (stage * STAGE_BYTES + BLOCK_BYTES))
            for i in range(LOADS):
                out.append("buffer_load_dwordx4 v%d, %%[vrsrc], 0 offen%s lds" %
                           (r.FTMP[LOADS + i], " offset:%d" % (1024 * i) if i else ""))
        if spread:
            return out
        for text in out:
            e(text)
            if text.startswith("s_add_u32 m0"):
                e("s_nop 0")
        return []

    def step_barrier(self, outstanding=2 * 2 * LOADS, spread=False):
        """Starts step s = tcount: unit s-1 has landed for every wave, everyone is
        done with unit s-2, whose stage takes unit s+2."""
        e = self.emit
        e("s_waitcnt vmcnt(%d)" % outstanding)
        e("s_barrier")
        e("s_add_u32 %[t2], %[tcount], 2")
        e("s_and_b32 %%[t2], %%[t2], %d" % (STAGES - 1))
        e("s_mul_i32 %%[t2], %%[t2], %d" % STAGE_BYTES)
        e("s_add_u32 %[tcount], %[tcount], 1")
        return self.request(spread=spread)

    def stage_addresses(self, k_part=True, v_part=True):
        """Read addresses of unit tcount - 2 (the step just started is tcount - 1)."""
        r = self.r
        e = self.emit
        e("s_add_u32 %[t0], %[tcount], 2")      # (tcount - 2) mod 4
        e("s_and_b32 %%[t0], %%[t0], %d" % (STAGES - 1))
        e("s_mul_i32 %%[t0], %%[t0], %d" % STAGE_BYTES)
        e("s_add_u32 %[t0], %[t0], %[ldsbase]")
        if k_part:
            for j in range(4):
                e("v_add_u32 v%d, %%[t0], v%d" % (r.KDYN[j], r.KADDR[j]))
        if v_part:
            for j in range(2):
                e("v_add_u32 v%d, %%[t0], v%d" % (r.VDYN[j], r.VADDR[j]))

    # ---- softmax of one block as a list of vector-side items ----------------------------------------------
    def softmax_items(self, parity, rare_label, resume_label, masked):
        r = self.r
        S = r.S[parity]
        PF = r.PF[parity]
        items = []
        if masked:
            for i in range(16):
                items.append("v_cmp_gt_i32 vcc, %d, v%d" % (8 * (i // 4) + i % 4, r.LIM))
                items.append("v_cndmask_b32 v%d, v%d, v%d, vcc" % (S + i, S + i, r.KMASK))
        items.append("v_max3_f32 v%d, v%d, v%d, v%d" % (r.T0, S, S + 1, S + 2))
        for i in range(3, 15, 2):
            items.append("v_max3_f32 v%d, v%d, v%d, v%d" % (r.T0, r.T0, S + i, S + i + 1))
        items.append("v_max_f32 v%d, v%d, v%d" % (r.T0, r.T0, S + 15))
        items.append("v_mov_b32 v%d, v%d" % (r.T1, r.T0))
        items.append("s_nop 1\n\tv_permlane32_swap_b32 v%d, v%d\n\ts_nop 1" % (r.T0, r.T1))
        items.append("v_max3_f32 v%d, v%d, v%d, v%d" % (r.MTRUE, r.MTRUE, r.T0, r.T1))
        items.append("v_mul_f32 v%d, %%[scale2], v%d" % (r.T0, r.MTRUE))
        items.append("v_cmp_gt_f32 vcc, v%d, v%d" % (r.T0, r.THR))
        items.append("s_cbranch_vccnz %s\n%s:" % (rare_label, resume_label))
        order = []
        for e in range(8):
            a, b = 2 * e, 2 * e + 1
            order += [("fma", a), ("fma", b), ("exp", a), ("exp", b)]
            if e > 0:
                order.append(("cvt", e - 1))
        order.append(("cvt", 7))
        for kind, i in order:
            if kind == "fma":
                items.append("v_fma_f32 v%d, v%d, %%[scale2], -v%d" % (S + i, S + i, r.MUSED))
            elif kind == "exp":
                items.append("v_exp_f32 v%d, v%d" % (S + i, S + i))
            else:
                s2, e = divmod(i, 4)
                items.append("v_cvt_pk_bf16_f32 v%d, v%d, v%d" %
                             (PF[s2] + e, S + 2 * i, S + 2 * i + 1))
        return items

    def rare_path(self, rare_label, resume_label):
        r = self.r
        e = self.emit
        e("%s:" % rare_label)
        e("v_cndmask_b32 v%d, v%d, v%d, vcc" % (r.T1, r.MUSED, r.T0))
        e("v_sub_f32 v%d, v%d, v%d" % (r.ALPHA, r.MUSED, r.T1))
        e("v_exp_f32 v%d, v%d" % (r.ALPHA, r.ALPHA))
        e("v_mov_b32 v%d, v%d" % (r.MUSED, r.T1))
        e("v_add_f32 v%d, 0x41000000, v%d" % (r.THR, r.T1))   # + 8.0
        e("s_mov_b32 %[flag], 1")
        e("s_branch %s" % resume_label)

    def rescale_path(self, label, resume_label):
        """Out of line, after the matrix instructions of block b-1 have been
        issued: accumulators follow the new reference point.  O^T goes through
        vector registers, four at a time."""
        r = self.r
        e = self.emit
        e("%s:" % label)
        e("s_nop 15")
        e("s_nop 15")
        for i in range(16):
            e("v_mul_f32 v%d, v%d, v%d" % (r.L + i, r.L + i, r.ALPHA))
        for first in range(0, 16 * DB, 4):
            for i in range(4):
                e("v_accvgpr_read_b32 v%d, a%d" % (r.RT[i], first + i))
            for i in range(4):
                e("v_mul_f32 v%d, v%d, v%d" % (r.RT[i], r.RT[i], r.ALPHA))
            for i in range(4):
                e("v_accvgpr_write_b32 a%d, v%d" % (first + i, r.RT[i]))
        e("s_mov_b32 %[flag], 0")
        e("s_nop 7")
        e("s_branch %s" % resume_label)

    # ---- one iteration ---------------------------------------------------------------------------------------
    def iteration(self, parity, scores, accumulate, softmax, masked, read_k, out_of_line,
                  requests=()):
        """Block b with b % 2 == parity.  scores: S^T(b+1) into S[1 - parity] from the
        K operands in OP.  accumulate: block b-1 from PF[1 - parity] and the V^T
        operands read here.  read_k: fetch the K operands of block b+2.  Both
        reads use the addresses stage_addresses() has set."""
        r = self.r
        slots = []
        if scores:
            slots += [("S", ks) for ks in range(KS)]
        if accumulate:
            for s2 in range(2):
                slots.append(("L", s2))
                slots += [("PV", s2, db) for db in range(DB)]
        items = []
        if softmax:
            rare, resume = self.label("rare"), self.label("resume")
            items = self.softmax_items(parity, rare, resume, masked)
            out_of_line.append(("rare", rare, resume))
        requests = list(requests)
        if not slots:
            for text in requests:
                self.emit(text)
                if text.startswith("s_add_u32 m0"):
                    self.emit("s_nop 0")
            for text in items:
                self.emit(text)
            return
        per_slot = (len(items) + len(slots) - 1) // len(slots)
        # one request every `stride` matrix instructions, from the second on
        stride = max(1, (len(slots) - 1) // max(len(requests), 1))
        if not scores and accumulate:
            for j in range(KS):
                self.v_read(j)
        at_item = 0
        for number, slot in enumerate(slots, 1):
            if slot[0] == "S":
                ks = slot[1]
                self.wait_for(("op", ks))
                acc = vt(r.S[1 - parity], 16)
                self.emit("%s %s, %s, %s, %s" % (MFMA, acc, vt(r.OP[ks], 4), at(r.QF[ks], 4),
                                                 "0" if ks == 0 else acc))
                if accumulate:
                    self.v_read(ks)
                elif read_k:
                    self.k_read(ks)
            elif slot[0] == "L":
                s2 = slot[1]
                acc = vt(r.L, 16)
                self.emit("%s %s, %s, %s, %s" % (MFMA, acc, vt(r.ONES, 4),
                                                 vt(r.PF[1 - parity][s2], 4), acc))
            else:
                s2, db = slot[1], slot[2]
                j = s2 * DB + db
                self.wait_for(("op", j))
                acc = at(r.O[db], 16)
                self.emit("%s %s, %s, %s, %s" % (MFMA, acc, vt(r.OP[j], 4),
                                                 vt(r.PF[1 - parity][s2], 4), acc))
                if read_k and scores:
                    self.k_read(j)
            for text in items[at_item:at_item + per_slot]:
                self.emit(text)
            at_item += per_slot
            if requests and number % stride == 0:
                self.emit(requests.pop(0))
        for text in requests:
            self.emit(text)
            if text.startswith("s_add_u32 m0"):
                self.emit("s_nop 0")
        for text in items[at_item:]:
            self.emit(text)
        if softmax and accumulate:
            label, back = self.label("rescale"), self.label("rescaled")
            self.emit("s_cmp_lg_u32 %[flag], 0")
            self.emit("s_cbranch_scc1 %s" % label)
            self.emit("%s:" % back)
            out_of_line.append(("rescale", label, back))

    def set_limit(self):
        """LIM for the block of the step just started (block tcount - 1 ... of the
        wave: its index is %[bcount])."""
        r = self.r
        e = self.emit
        e("s_lshl_b32 %[t1], %[bcount], 5")
        e("v_subrev_u32 v%d, %%[t1], v%d" % (r.LIM, r.ROWLIM))

    # ---- the whole statement ---------------------------------------------------------------------------------
    def build(self):
        r = self.r
        e = self.emit
        out_of_line = []
        e("s_mov_b32 %[m0save], m0")
        e("s_waitcnt lgkmcnt(0)")
        # K(0), K(1), K(2) into the K halves of stages 1, 2, 3 (units -3, -2, -1), while Q is
        # still on its way; then Q^T to AGPRs, O^T to zero
        for stage in (1, 2, 3):
            self.request(stage=stage, v_part=False)
        e("s_waitcnt vmcnt(%d)" % (3 * LOADS))
        for ks in range(KS):
            for i in range(4):
                e("v_accvgpr_write_b32 a%d, v%d" % (r.QF[ks] + i, r.QIN[ks] + i))
        for i in range(16 * DB):
            e("v_accvgpr_write_b32 a%d, 0" % i)
        e("v_mov_b32 v%d, 0xff7fffff" % r.KMASK)
        # tcount counts steps from -2: the uniform rule (step s: unit s-1 landed, request unit s+2
        # into stage (s+2) mod 4, read addresses of unit s-1 = stage (s+3) mod 4) holds from there,
        # with fewer requests in flight at the first two
        e("s_mov_b32 %[tcount], -2")
        # step -2: K(0) (unit -3) landed; request unit 0 = {K(3), V(0)}
        self.step_barrier(outstanding=2 * LOADS)
        self.stage_addresses(v_part=False)
        for ks in range(KS):
            self.k_read(ks)
        # step -1: K(1) landed; S^T(0), and the K operands of block 1 into the registers it leaves.
        # The barrier lets unit 1 into the stage of K(0): its reads have returned.
        self.wait_for(("op", KS - 1))
        self.step_barrier(outstanding=LOADS + 2 * LOADS)
        self.stage_addresses(v_part=False)
        self.iteration(1, True, False, False, False, True, out_of_line)
        e("s_nop 15")   # S^T(0) has left the matrix pipe before the vector side reads it
        e("s_mov_b32 %[bcount], 0")
        one, two, loop, idle = "Lone_%=", "Ltwo_%=", "Lloop_%=", "Lidle_%="
        tail = {1: "Ltail_odd_%=", 0: "Ltail_even_%="}    # by the parity of block nblk - 2
        last = {1: "Llast_odd_%=", 0: "Llast_even_%="}    # by the parity of block nblk - 1
        e("s_cmp_eq_u32 %[nblk], 1")
        e("s_cbranch_scc1 %s" % one)
        # iteration 0: softmax(0), S^T(1); K operands of block 2
        requests = self.step_barrier(spread=True)
        self.stage_addresses(v_part=False)
        self.set_limit()
        self.iteration(0, True, False, True, True, True, out_of_line, requests=requests)
        e("s_mov_b32 %[flag], 0")   # a reference point that moved before anything was accumulated
        e("s_mov_b32 %[bcount], 1")
        e("s_cmp_eq_u32 %[nblk], 2")
        e("s_cbranch_scc1 %s" % two)
        # steady state: iterations b = 1 .. nblk - 3
        e("%s:" % loop)
        at_loop_top = list(self.lds_queue)
        for parity in (1, 0):
            e("s_cmp_eq_u32 %[iters], 0")
            e("s_cbranch_scc1 %s" % tail[parity])
            requests = self.step_barrier(spread=True)
            self.stage_addresses()
            self.iteration(parity, True, True, True, False, True, out_of_line, requests=requests)
            e("s_sub_u32 %[iters], %[iters], 1")
            e("s_add_u32 %[bcount], %[bcount], 1")
            assert self.lds_queue == at_loop_top, (self.lds_queue, at_loop_top)
        e("s_branch %s" % loop)
        # a wave's last two blocks (masks) and the products still owed
        for p in (1, 0):
            e("%s:" % tail[p])
            self.lds_queue = list(at_loop_top)
            # block nblk - 2: S^T of the last block, no further K operands
            requests = self.step_barrier(spread=True)
            self.stage_addresses()
            self.set_limit()
            self.iteration(p, True, True, True, True, False, out_of_line, requests=requests)
            e("s_add_u32 %[bcount], %[bcount], 1")
            assert self.lds_queue == []
            e("%s:" % last[1 - p])
            # block nblk - 1 (parity 1 - p): softmax and the products of block nblk - 2
            requests = self.step_barrier(spread=True)
            self.stage_addresses(k_part=False)
            self.set_limit()
            self.iteration(1 - p, False, True, True, True, False, out_of_line, requests=requests)
            # the products of block nblk - 1
            requests = self.step_barrier(spread=True)
            self.stage_addresses(k_part=False)
            e("s_nop 7")
            self.iteration(p, False, True, False, False, False, out_of_line, requests=requests)
            assert self.lds_queue == []
            e("s_branch %s" % idle)
        # a wave with two blocks: block 1 is its last (the K operands requested for a
        # block 2 are awaited so that the reads in flight are the ones counted)
        e("%s:" % two)
        e("s_waitcnt lgkmcnt(0)")
        e("s_branch %s" % last[1])
        # a wave with a single block
        e("%s:" % one)
        e("s_waitcnt lgkmcnt(0)")
        self.lds_queue = []
        self.step_barrier()
        self.set_limit()
        self.iteration(0, False, False, True, True, False, out_of_line)
        requests = self.step_barrier(spread=True)
        self.stage_addresses(k_part=False)
        e("s_nop 7")
        self.iteration(1, False, True, False, False, False, out_of_line, requests=requests)
        # the steps the slowest wave still has to take: barriers and requests only
        e("%s:" % idle)
        again, finished = "Lidle_again_%=", "Lfinished_%="
        e("%s:" % again)
        e("s_cmp_eq_u32 %[idle], 0")
        e("s_cbranch_scc1 %s" % finished)
        self.step_barrier()
        e("s_sub_u32 %[idle], %[idle], 1")
        e("s_branch %s" % again)
        e("%s:" % finished)
        e("s_waitcnt vmcnt(0) lgkmcnt(0)")
        e("s_nop 15")
        e("s_nop 15")
        e("s_barrier")
        for db in range(DB):
            for i in range(16):
                e("v_accvgpr_read_b32 v%d, a%d" % (r.OUT[db] + i, r.O[db] + i))
        e("s_mov_b32 m0, %[m0save]")
        end = "Lend_%="
        e("s_branch %s" % end)
        for kind, label, back in out_of_line:
            if kind == "rare":
                self.rare_path(label, back)
            else:
                self.rescale_path(label, back)
        e("%s:" % end)


def c_string(lines, indent="  "):
    return "\n".join('%s"%s\\n\\t"' % (indent, line.replace("\n", "\\n").replace("\t", "\\t"))
                     for line in lines)


def render():
    g = Emitter()
    g.build()
    r = g.r
    name = "FLASH_LOOP_D256"
    out = ["// head width 256, %d waves a workgroup: %d instructions and labels" % (WAVES, len(g.lines))]
    out.append("#define %s_ASM \\" % name)
    out.append(" \\\n".join(c_string(g.lines).split("\n")))
    out.append("")

    def define(tag, value):
        out.append("#define %s_%s %s" % (name, tag, value))

    for db in range(DB):
        define("O%d" % db, '"=&{%s}"' % vt(r.OUT[db], 16))
    define("L", '"+{%s}"' % vt(r.L, 16))
    for ks in range(KS):
        define("QF%d" % ks, '"+{%s}"' % vt(r.QIN[ks], 4))
    define("ONES", '"{%s}"' % vt(r.ONES, 4))
    for j in range(4):
        define("KADDR%d" % j, '"{v%d}"' % r.KADDR[j])
    for j in range(2):
        define("VADDR%d" % j, '"{v%d}"' % r.VADDR[j])
    for i in range(LOADS):
        define("KFILL%d" % i, '"{v%d}"' % r.KFILL[i])
        define("VFILL%d" % i, '"{v%d}"' % r.VFILL[i])
    define("MUSED", '"+{v%d}"' % r.MUSED)
    define("MTRUE", '"+{v%d}"' % r.MTRUE)
    define("THR", '"+{v%d}"' % r.THR)
    define("ROWLIM", '"{v%d}"' % r.ROWLIM)
    clobbers = ['"v%d"' % v for v in range(r.pinned_end, r.temps_end)]
    clobbers += ['"a%d"' % a for a in range(r.agprs)]
    define("CLOBBERS", ", ".join(clobbers) + ', "vcc", "scc", "memory"')
    define("LOADS", str(LOADS))
    define("WAVES", str(WAVES))
    define("STAGE_BYTES", str(STAGE_BYTES))
    define("BLOCK_BYTES", str(BLOCK_BYTES))
    return "\n".join(out) + "\n"


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    target = sys.argv[1] if len(sys.argv) > 1 else os.path.join(here, "flash_fwd_loop256.inc")
    text = ("// Generated by gen_flash_fwd_loop256.py; do not edit.  The instruction stream of the\n"
            "// main loop of flash_forward_pipelined_kernel<256>, see the generator for the schedule.\n\n")
    text += render()
    with open(target, "w") as f:
        f.write(text)


if __name__ == "__main__":
    main()
