#!/usr/bin/env python3
"""Writes flash_fwd_loop.inc: the hand-scheduled gfx950 instruction stream of
the causal flash-attention forward kernel's main loop (flash_fwd_pipelined.hip),
one text per head width, as the body of a single `asm volatile` statement with
a fixed register allocation.

Why generated text and not C++: what bounds the loop is instruction issue.  A
wave that alternates bursts of matrix instructions with bursts of softmax
arithmetic leaves the matrix pipe idle half of the time; a wave whose matrix
instructions are each followed by two or three vector instructions and an LDS
read keeps it busy (measured on the part: 16 MFMA + the softmax mix of one
32-key block, interleaved, take the time of the 16 MFMA alone).  The compiler's
scheduler does not produce that order, so the order is written here:

  iteration b (one 32-key block) issues, interleaved,
    matrix:  S^T(b+1) = K(b+1) Q^T            KS instructions
             l, O^T  += [1; V^T(b-1)] P^T(b-1)   2 (1 + DB) instructions
    vector:  softmax of block b: running maximum, P^T(b) = 2^(S^T(b) c - m) as bf16
    LDS:     V^T operands of block b-1 (into the registers the K operands of
             block b+1 have just left), K operands of block b+2 (into the
             registers the V^T operands leave)
  so that no instruction waits for a result of the same iteration.

K/V tiles of 64 keys travel global -> LDS in units {K(u+1), V(u)} through a
ring of four stages; a workgroup barrier per unit (two iterations) hands a
stage over.  Units are requested two barriers before they are read.

The text uses named operands (%[name]) for scalar inputs and physical vector
registers, which the enclosing statement pins with "{v[a:b]}" constraints and
lists as clobbers; FLASH_LOOP_*_REGS macros carry the numbers to the C++ side.

Usage: python gen_flash_fwd_loop.py [output]   (default: flash_fwd_loop.inc
beside this file)
"""
import os
import sys


class Registers:
    """Vector register map, allocated from v255 downwards."""

    def __init__(self, D, waves):
        self.D = D
        self.waves = waves
        self.KS = D // 16          # contraction steps of S^T = operand tuples
        self.DB = D // 32          # 32-channel blocks of O^T
        top = 256

        def take(n, align=4):
            nonlocal top
            top -= n
            top -= top % align
            return top

        self.O = [take(16, 16) for _ in range(self.DB)]
        self.O.reverse()
        self.L = take(16, 16)
        self.S = [take(16, 16), take(16, 16)]
        self.QF = [take(4) for _ in range(self.KS)]
        self.QF.reverse()
        self.OP = [take(4) for _ in range(self.KS)]
        self.OP.reverse()
        self.PF = [[take(4), take(4)], [take(4), take(4)]]   # [parity][s2]
        self.ONES = take(4)
        self.two_bases = 4 * self.stage_bytes() > 65536
        self.KADDR = [[take(1, 1) for _ in range(self.KS)]]
        self.VADDR = [[take(1, 1) for _ in range(self.DB)]]
        if self.two_bases:
            self.KADDR.append([take(1, 1) for _ in range(self.KS)])
            self.VADDR.append([take(1, 1) for _ in range(self.DB)])
        self.loads = 64 * (D // 8) // (64 * waves)  # 16-byte loads a lane, tensor and tile
        self.KFILL = [take(1, 1) for _ in range(self.loads)]
        self.VFILL = [take(1, 1) for _ in range(self.loads)]
        self.FTMP = [take(1, 1) for _ in range(2 * self.loads)]
        self.MUSED = take(1, 1)
        self.MTRUE = take(1, 1)
        self.THR = take(1, 1)
        self.T0 = take(1, 1)
        self.T1 = take(1, 1)
        self.ALPHA = take(1, 1)
        self.DADDR = [take(1, 1) for _ in range(self.DB)]   # V^T read addresses of the last blocks
        self.LIM = take(1, 1)      # last key offset a lane's query sees in the block at hand
        self.KMASK = take(1, 1)    # the finite sentinel of masked scores
        self.ROWLIM = take(1, 1)   # input: last key the lane's query sees, minus 4 h
        self.lowest = top

    def tile_bytes(self):
        return 64 * self.D * 2

    def stage_bytes(self):
        return 2 * self.tile_bytes()

    def half_bytes(self):
        return 32 * self.D * 2

    def row_bytes(self):
        return self.D * 2


def vt(base, n):
    return "v[%d:%d]" % (base, base + n - 1) if n > 1 else "v%d" % base


class Emitter:
    def __init__(self, D, waves):
        self.r = Registers(D, waves)
        self.lines = []
        self.label_count = 0
        self.lds_queue = []     # destination tuples of LDS reads in flight, oldest first

    # ---- text ---------------------------------------------------------------
    def emit(self, text):
        self.lines.append(text)

    def label(self, stem):
        self.label_count += 1
        return "L%s_%d_%%=" % (stem, self.label_count)

    # ---- LDS reads with lgkmcnt bookkeeping ------------------------------------
    def lds_read(self, text, dest):
        self.emit(text)
        self.lds_queue.append(dest)

    def wait_for(self, dest):
        """s_waitcnt so that every queued read into `dest` has returned (LDS
        reads return in order)."""
        last = -1
        for i, d in enumerate(self.lds_queue):
            if d == dest:
                last = i
        if last < 0:
            return
        younger = len(self.lds_queue) - 1 - last
        assert younger <= 15, "lgkmcnt holds four bits"
        self.emit("s_waitcnt lgkmcnt(%d)" % younger)
        self.lds_queue = self.lds_queue[last + 1:]

    def k_read(self, j, stage, half):
        r = self.r
        offset = stage * r.stage_bytes() + half * r.half_bytes()
        base = r.KADDR[0][j]
        if offset >= 65536:
            base = r.KADDR[1][j]
            offset -= 65536
        self.lds_read("ds_read_b128 %s, v%d offset:%d" % (vt(r.OP[j], 4), base, offset), ("op", j))

    def v_read(self, j, stage, half, address=None):
        """V^T operand tuple j = (s2, db): two transposing reads."""
        r = self.r
        s2, db = divmod(j, r.DB)
        offset = r.tile_bytes() + half * r.half_bytes() + 16 * s2 * r.row_bytes()
        if address is None:
            offset += stage * r.stage_bytes()
            base = r.VADDR[0][db]
            if offset + 8 * r.row_bytes() >= 65536:
                base = r.VADDR[1][db]
                offset -= 65536
        else:
            base = address[db]
        self.lds_read("ds_read_b64_tr_b16 %s, v%d offset:%d" % (vt(r.OP[j], 2), base, offset),
                      ("op", j))
        self.lds_read("ds_read_b64_tr_b16 %s, v%d offset:%d" %
                      (vt(r.OP[j] + 2, 2), base, offset + 8 * r.row_bytes()), ("op", j))

    # ---- global -> LDS fills -----------------------------------------------------
    def fill(self, stage, k_part=True, v_part=True, advance=True):
        """Requests K rows at byte offset %[koff] and V rows at %[voff] into a
        stage; 2 * loads (or loads) vector-memory operations a wave."""
        r = self.r
        n = r.loads
        if k_part:
            for i in range(n):
                self.emit("v_add_u32 v%d, %%[koff], v%d" % (r.FTMP[i], r.KFILL[i]))
        if v_part:
            for i in range(n):
                self.emit("v_add_u32 v%d, %%[voff], v%d" % (r.FTMP[n + i], r.VFILL[i]))
        if k_part:
            self.emit("s_add_u32 m0, %%[ldsw], %d" % (stage * r.stage_bytes()))
            self.emit("s_nop 0")
            for i in range(n):
                self.emit("buffer_load_dwordx4 v%d, %%[krsrc], 0 offen%s lds" %
                          (r.FTMP[i], " offset:%d" % (1024 * i) if i else ""))
        if v_part:
            self.emit("s_add_u32 m0, %%[ldsw], %d" % (stage * r.stage_bytes() + r.tile_bytes()))
            self.emit("s_nop 0")
            for i in range(n):
                self.emit("buffer_load_dwordx4 v%d, %%[vrsrc], 0 offen%s lds" %
                          (r.FTMP[n + i], " offset:%d" % (1024 * i) if i else ""))
        if advance:
            if k_part:
                self.emit("s_add_u32 %[koff], %[koff], %[kstep]")
            if v_part:
                self.emit("s_add_u32 %[voff], %[voff], %[vstep]")

    # ---- the softmax of one block as a list of vector-side items ------------------------
    def softmax_items(self, parity, rare_label, resume_label, masked=False):
        r = self.r
        S = r.S[parity]
        PF = r.PF[parity]
        items = []
        if masked:
            # register i holds key 8 (i / 4) + i % 4 (+ 4 h, folded into LIM) of the block;
            # keys beyond the lane's limit get the finite sentinel of the reference kernels
            for i in range(16):
                items.append("v_cmp_gt_i32 vcc, %d, v%d" % (8 * (i // 4) + i % 4, r.LIM))
                items.append("v_cndmask_b32 v%d, v%d, v%d, vcc" % (S + i, S + i, r.KMASK))
        # running maximum: the order of flash_forward_kernel
        items.append("v_max3_f32 v%d, v%d, v%d, v%d" % (r.T0, S, S + 1, S + 2))
        for i in range(3, 15, 2):
            items.append("v_max3_f32 v%d, v%d, v%d, v%d" % (r.T0, r.T0, S + i, S + i + 1))
        items.append("v_max_f32 v%d, v%d, v%d" % (r.T0, r.T0, S + 15))
        items.append("v_mov_b32 v%d, v%d" % (r.T1, r.T0))
        # both lane halves of a query: T0 <- lower halves' values, T1 <- upper halves'
        items.append("s_nop 1\n\tv_permlane32_swap_b32 v%d, v%d\n\ts_nop 1" % (r.T0, r.T1))
        items.append("v_max3_f32 v%d, v%d, v%d, v%d" % (r.MTRUE, r.MTRUE, r.T0, r.T1))
        items.append("v_mul_f32 v%d, %%[scale2], v%d" % (r.T0, r.MTRUE))
        items.append("v_cmp_gt_f32 vcc, v%d, v%d" % (r.T0, r.THR))
        items.append("s_cbranch_vccnz %s\n%s:" % (rare_label, resume_label))
        # P^T = 2^(S^T scale2 - m_used), packed to bf16 pairs as they complete
        order = []
        for e in range(8):
            a, b = 2 * e, 2 * e + 1
            order.append(("fma", a))
            order.append(("fma", b))
            order.append(("exp", a))
            order.append(("exp", b))
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
        """Out of line: the reference point of the online softmax moves for some
        row.  T0 holds the candidate, vcc the rows whose maximum outgrew it."""
        r = self.r
        self.emit("%s:" % rare_label)
        self.emit("v_cndmask_b32 v%d, v%d, v%d, vcc" % (r.T1, r.MUSED, r.T0))
        self.emit("v_sub_f32 v%d, v%d, v%d" % (r.ALPHA, r.MUSED, r.T1))
        self.emit("v_exp_f32 v%d, v%d" % (r.ALPHA, r.ALPHA))
        self.emit("v_mov_b32 v%d, v%d" % (r.MUSED, r.T1))
        self.emit("v_add_f32 v%d, 0x41000000, v%d" % (r.THR, r.T1))   # + 8.0
        self.emit("s_mov_b32 %[flag], 1")
        self.emit("s_branch %s" % resume_label)

    def rescale_path(self, label, resume_label):
        """Out of line, after the matrix instructions of block b-1 have been
        issued: accumulators follow the new reference point."""
        r = self.r
        self.emit("%s:" % label)
        self.emit("s_nop 15")
        self.emit("s_nop 15")
        self.emit("v_mul_f32 v%d, v%d, v%d" % (r.L, r.L, r.ALPHA))
        for base in r.O:
            for i in range(16):
                self.emit("v_mul_f32 v%d, v%d, v%d" % (base + i, base + i, r.ALPHA))
        self.emit("s_mov_b32 %[flag], 0")
        self.emit("s_nop 3")
        self.emit("s_branch %s" % resume_label)

    # ---- one iteration -----------------------------------------------------------------
    def iteration(self, parity, scores=True, accumulate=True, softmax=True, v_from=None,
                  k_from=None, drain_address=None, out_of_line=None, masked=False, requests=()):
        """Block b with b % 2 == parity.  scores: S^T(b+1) into S[1 - parity] from
        the K operands in OP.  accumulate: block b-1 from PF[1 - parity] and the
        V^T operands read here from v_from = (stage, half).  k_from: where the K
        operands of block b+2 come from.  out_of_line collects the rare paths."""
        r = self.r
        KS, DB = r.KS, r.DB
        slots = []
        if scores:
            slots += [("S", ks) for ks in range(KS)]
        if accumulate:
            for s2 in range(2):
                slots.append(("L", s2))
                slots += [("PV", s2, db) for db in range(DB)]
        items = []
        rescale_label = None
        if softmax:
            rare, resume = self.label("rare"), self.label("resume")
            items = self.softmax_items(parity, rare, resume, masked)
            out_of_line.append(("rare", rare, resume))
        if not slots:
            for text in items:
                self.emit(text)
            return
        per_slot = (len(items) + len(slots) - 1) // len(slots)
        if not scores and accumulate:
            # no S^T products to hide the V^T reads behind: request them up front
            for j in range(KS):
                self.v_read(j, v_from[0] if v_from else 0, v_from[1] if v_from else 0,
                            drain_address)
        at = 0
        requests = list(requests)
        stride = max(1, (len(slots) - 1) // max(len(requests), 1))
        for number, slot in enumerate(slots, 1):
            if slot[0] == "S":
                ks = slot[1]
                self.wait_for(("op", ks))
                acc = vt(r.S[1 - parity], 16)
                self.emit("v_mfma_f32_32x32x16_bf16 %s, %s, %s, %s" %
                          (acc, vt(r.OP[ks], 4), vt(r.QF[ks], 4), "0" if ks == 0 else acc))
                if accumulate:
                    self.v_read(ks, v_from[0], v_from[1], drain_address)
                elif k_from is not None:
                    self.k_read(ks, k_from[0], k_from[1])
            elif slot[0] == "L":
                s2 = slot[1]
                acc = vt(r.L, 16)
                self.emit("v_mfma_f32_32x32x16_bf16 %s, %s, %s, %s" %
                          (acc, vt(r.ONES, 4), vt(r.PF[1 - parity][s2], 4), acc))
            else:
                s2, db = slot[1], slot[2]
                j = s2 * DB + db
                self.wait_for(("op", j))
                acc = vt(r.O[db], 16)
                self.emit("v_mfma_f32_32x32x16_bf16 %s, %s, %s, %s" %
                          (acc, vt(r.OP[j], 4), vt(r.PF[1 - parity][s2], 4), acc))
                if k_from is not None and scores:
                    self.k_read(j, k_from[0], k_from[1])
            for text in items[at:at + per_slot]:
                self.emit(text)
            at += per_slot
            if requests and number % stride == 0:
                self.emit(requests.pop(0))
        for text in requests:
            self.emit(text)
            if text.startswith("s_add_u32 m0"):
                self.emit("s_nop 0")
        for text in items[at:]:
            self.emit(text)
        if softmax and accumulate:
            rescale_label, back = self.label("rescale"), self.label("rescaled")
            self.emit("s_cmp_lg_u32 %[flag], 0")
            self.emit("s_cbranch_scc1 %s" % rescale_label)
            self.emit("%s:" % back)
            out_of_line.append(("rescale", rescale_label, back))

    def step_barrier(self, spread=False):
        """The barrier that starts step t (before odd iteration 2t-1): unit t has
        landed for every wave, everyone is done with unit t-2, whose stage takes
        unit t+2.  The stage is computed, so the same text serves every place.
        With `spread` the requests are returned instead of emitted, for the
        iteration that follows to deal out between its matrix instructions: the
        waves of a workgroup leave the barrier together, and requests issued
        there queue behind each other at the compute unit's one address path
        while nothing else is issued."""
        r = self.r
        n = r.loads
        e = self.emit
        e("s_waitcnt vmcnt(%d)" % (2 * n))
        e("s_barrier")
        e("s_add_u32 %[tcount], %[tcount], 1")
        e("s_add_u32 %[t0], %[tcount], 2")
        e("s_and_b32 %[t0], %[t0], 3")
        e("s_mul_i32 %%[t0], %%[t0], %d" % r.stage_bytes())
        e("s_add_u32 %[t0], %[t0], %[ldsw]")
        for i in range(n):
            e("v_add_u32 v%d, %%[koff], v%d" % (r.FTMP[i], r.KFILL[i]))
        for i in range(n):
            e("v_add_u32 v%d, %%[voff], v%d" % (r.FTMP[n + i], r.VFILL[i]))
        e("s_mov_b32 m0, %[t0]")
        e("s_add_u32 %[koff], %[koff], %[kstep]")
        e("s_add_u32 %[voff], %[voff], %[vstep]")
        requests = []
        for i in range(n):
            requests.append("buffer_load_dwordx4 v%d, %%[krsrc], 0 offen%s lds" %
                            (r.FTMP[i], " offset:%d" % (1024 * i) if i else ""))
        requests.append("s_add_u32 m0, m0, %d" % r.tile_bytes())
        for i in range(n):
            requests.append("buffer_load_dwordx4 v%d, %%[vrsrc], 0 offen%s lds" %
                            (r.FTMP[n + i], " offset:%d" % (1024 * i) if i else ""))
        if spread:
            return requests
        for text in requests:
            e(text)
            if text.startswith("s_add_u32 m0"):
                e("s_nop 0")
        return []

    def last_block_setup(self, masked):
        """Before one of a wave's last iterations, which read V^T of block
        %[vblk] from computed addresses and (masked) work on block vblk + 1."""
        r = self.r
        e = self.emit
        # V block j sits in unit j / 2: stage (j / 2) % 4, half j % 2
        e("s_lshr_b32 %[t0], %[vblk], 1")
        e("s_and_b32 %[t0], %[t0], 3")
        e("s_mul_i32 %%[t0], %%[t0], %d" % r.stage_bytes())
        e("s_and_b32 %[t1], %[vblk], 1")
        e("s_mul_i32 %%[t1], %%[t1], %d" % r.half_bytes())
        e("s_add_u32 %[t0], %[t0], %[t1]")
        for db in range(r.DB):
            e("v_add_u32 v%d, %%[t0], v%d" % (r.DADDR[db], r.VADDR[0][db]))
        if masked:
            e("s_add_u32 %[t1], %[vblk], 1")
            e("s_lshl_b32 %[t1], %[t1], 5")
            e("v_subrev_u32 v%d, %%[t1], v%d" % (r.LIM, r.ROWLIM))

    # ---- the whole statement ------------------------------------------------------------
    def build(self):
        r = self.r
        out_of_line = []
        e = self.emit
        n = r.loads
        one, drain_odd, pre_odd, pre_even, idle = ("Lone_%=", "Ldrain_odd_%=", "Lpre_odd_%=",
                                                   "Lpre_even_%=", "Lidle_%=")
        e("s_mov_b32 %[m0save], m0")
        e("s_waitcnt vmcnt(0)")
        e("v_mov_b32 v%d, 0xff7fffff" % r.KMASK)
        # ---- prologue: K(0) into the K half of stage 3, units 0..2; K(0) and unit 0 awaited ----
        self.fill(3, v_part=False)
        for u in range(3):
            self.fill(u)
        e("s_waitcnt vmcnt(%d)" % (4 * n))
        e("s_barrier")
        for ks in range(r.KS):
            self.k_read(ks, 3, 0)
        # S^T(0), then the K operands of block 1 into the registers it leaves
        self.iteration(1, scores=True, accumulate=False, softmax=False, k_from=(3, 1),
                       out_of_line=out_of_line)
        e("s_nop 15")   # S^T(0) has left the matrix pipe before the vector side reads it
        e("v_mov_b32 v%d, v%d" % (r.LIM, r.ROWLIM))
        e("s_cmp_eq_u32 %[nblk], 1")
        e("s_cbranch_scc1 %s" % one)
        # iteration 0: softmax(0), S^T(1); K operands of block 2 = K(1), first half (unit 0)
        self.iteration(0, scores=True, accumulate=False, softmax=True, k_from=(0, 0),
                       out_of_line=out_of_line, masked=True)
        # a reference point that moved before anything was accumulated: O and l are zero
        e("s_mov_b32 %[flag], 0")
        e("s_cmp_eq_u32 %[nblk], 2")
        e("s_cbranch_scc1 %s" % drain_odd)
        # ---- steady state: iterations b = 1 .. nblk - 3, eight to a round (four units) --------
        loop = "Lloop_%="
        e("%s:" % loop)
        at_loop_top = list(self.lds_queue)
        for position in range(8):
            b = position + 1           # b mod 8
            t = (b + 1) // 2           # its step, mod 4 below
            e("s_cmp_eq_u32 %[iters], 0")
            e("s_cbranch_scc1 %s" % (pre_odd if b % 2 else pre_even))
            if b % 2:
                # odd iteration 2t-1: unit t-1 holds V(t-1) and K(t)
                requests = self.step_barrier(spread=True)
                self.iteration(1, v_from=((t - 1) % 4, 0), k_from=((t - 1) % 4, 1),
                               out_of_line=out_of_line, requests=requests)
            else:
                # even iteration 2t: V(t-1) second half; K(t+1) first half (unit t)
                self.iteration(0, v_from=((t - 1) % 4, 1), k_from=(t % 4, 0),
                               out_of_line=out_of_line)
            e("s_sub_u32 %[iters], %[iters], 1")
            e("s_add_u32 %[vblk], %[vblk], 1")
            # every way on leaves the same reads in flight
            assert self.lds_queue == at_loop_top
        e("s_branch %s" % loop)
        # ---- a wave's last two blocks (masks) and the products still owed -----------------------
        for first_odd in (True, False):
            e("%s:" % (pre_odd if first_odd else pre_even))
            self.lds_queue = list(at_loop_top)
            if first_odd:
                self.step_barrier()
            self.last_block_setup(masked=True)
            self.iteration(1 if first_odd else 0, scores=True, accumulate=True, softmax=True,
                           v_from=(0, 0), drain_address=r.DADDR, out_of_line=out_of_line,
                           masked=True)
            e("s_add_u32 %[vblk], %[vblk], 1")
            if not first_odd:
                e("%s:" % drain_odd)
                self.step_barrier()
            self.last_block_setup(masked=True)
            self.iteration(0 if first_odd else 1, scores=False, accumulate=True, softmax=True,
                           v_from=(0, 0), drain_address=r.DADDR, out_of_line=out_of_line,
                           masked=True)
            e("s_add_u32 %[vblk], %[vblk], 1")
            self.last_block_setup(masked=False)
            e("s_nop 7")
            self.iteration(1 if first_odd else 0, scores=False, accumulate=True, softmax=False,
                           v_from=(0, 0), drain_address=r.DADDR, out_of_line=out_of_line)
            e("s_branch %s" % idle)
        # ---- a wave with a single block ---------------------------------------------------------
        e("%s:" % one)
        self.iteration(0, scores=False, accumulate=False, softmax=True, out_of_line=out_of_line,
                       masked=True)
        self.last_block_setup(masked=False)
        e("s_nop 7")
        self.iteration(1, scores=False, accumulate=True, softmax=False, v_from=(0, 0),
                       drain_address=r.DADDR, out_of_line=out_of_line)
        # ---- the steps the slowest wave still has to take: barriers and fills only ------------
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
        e("s_mov_b32 m0, %[m0save]")
        end = "Lend_%="
        e("s_branch %s" % end)
        for kind, label, back in out_of_line:
            if kind == "rare":
                self.rare_path(label, back)
            else:
                self.rescale_path(label, back)
        e("%s:" % end)

    def text(self):
        return self.lines


def c_string(lines, indent="  "):
    return "\n".join('%s"%s\\n\\t"' % (indent, line.replace("\n", "\\n").replace("\t", "\\t"))
                     for line in lines)


def render(D, waves):
    g = Emitter(D, waves)
    g.build()
    r = g.r
    name = "FLASH_LOOP_D%d" % D
    out = []
    out.append("// head width %d, %d waves a workgroup: %d instructions and labels, vector registers "
               "v%d..v255" % (D, waves, len(g.lines), r.lowest))
    out.append("#define %s_ASM \\" % name)
    body = c_string(g.lines).split("\n")
    out.append(" \\\n".join(body))
    out.append("")

    def define(tag, value):
        out.append("#define %s_%s %s" % (name, tag, value))

    for db in range(r.DB):
        define("O%d" % db, '"+{%s}"' % vt(r.O[db], 16))
    define("L", '"+{%s}"' % vt(r.L, 16))
    for ks in range(r.KS):
        define("QF%d" % ks, '"{%s}"' % vt(r.QF[ks], 4))
    define("ONES", '"{%s}"' % vt(r.ONES, 4))
    for set_index, (ka, va) in enumerate(zip(r.KADDR, r.VADDR)):
        for ks in range(r.KS):
            define("KADDR%d_%d" % (set_index, ks), '"{v%d}"' % ka[ks])
        for db in range(r.DB):
            define("VADDR%d_%d" % (set_index, db), '"{v%d}"' % va[db])
    define("TWO_BASES", "1" if r.two_bases else "0")
    for i in range(r.loads):
        define("KFILL%d" % i, '"{v%d}"' % r.KFILL[i])
        define("VFILL%d" % i, '"{v%d}"' % r.VFILL[i])
    define("LOADS", str(r.loads))
    define("WAVES", str(waves))
    define("MUSED", '"+{v%d}"' % r.MUSED)
    define("MTRUE", '"+{v%d}"' % r.MTRUE)
    define("THR", '"+{v%d}"' % r.THR)
    define("ROWLIM", '"{v%d}"' % r.ROWLIM)
    pinned = set()
    for base in r.O + [r.L]:
        pinned.update(range(base, base + 16))
    for base in r.QF + [r.ONES]:
        pinned.update(range(base, base + 4))
    for group in r.KADDR + r.VADDR:
        pinned.update(group)
    pinned.update(r.KFILL + r.VFILL + [r.MUSED, r.MTRUE, r.THR, r.ROWLIM])
    clobbers = [v for v in range(r.lowest, 256) if v not in pinned]
    define("CLOBBERS", ", ".join('"v%d"' % v for v in clobbers) + ', "vcc", "scc", "memory"')
    define("LOWEST_VGPR", str(r.lowest))
    define("STAGE_BYTES", str(r.stage_bytes()))
    return "\n".join(out) + "\n"


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    target = sys.argv[1] if len(sys.argv) > 1 else os.path.join(here, "flash_fwd_loop.inc")
    text = ("// Generated by gen_flash_fwd_loop.py; do not edit.  The instruction stream of the\n"
            "// main loop of flash_forward_pipelined_kernel, see the generator for the schedule.\n\n")
    for D, waves in ((128, 8), (64, 4)):
        text += render(D, waves) + "\n"
    with open(target, "w") as f:
        f.write(text)


if __name__ == "__main__":
    main()
