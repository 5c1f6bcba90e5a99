"""Emitter for hand-scheduled gfx950 instruction streams placed in `asm volatile` statements.

Streams are written by generator scripts (gen_*_tile.py) as a sequence of MFMA, VALU and LDS
operations with explicit registers.  The emitter keeps the order it is given and inserts what the
hardware leaves to software on gfx950:
    MFMA (8 pass) result -> VALU / LDS / MFMA-A/B use     12 wait states
    VALU result          -> MFMA operand                   2 wait states
    transcendental result-> VALU use                        1 wait state
    dot (v_dot2c) result -> other VALU use / overwrite      4 wait states (accumulating dots chain freely)
    MFMA reading C from registers other than its destination -> VALU write of them   12 wait states
    fp32 MFMA (32x32x2, 16 pass) result -> any use                20 wait states
    LDS read result      -> any use                         s_waitcnt lgkmcnt (reads return in order)
Registers are ("v", n) / ("a", n) pairs, or any other hashable key a generator chooses for a
compiler-supplied operand it wants tracked (("op", name)).

Blocks that a scalar branch may skip (skip_begin / skip_end around them) are scheduled as if executed,
and the code behind them is scheduled for both cases: as if the block had taken no time, with the
block's register writes as recent as possible and the writes before the block still remembered.
"""


def vr(lo, n=1):
    return f"v{lo}" if n == 1 else f"v[{lo}:{lo + n - 1}]"


def ar(lo, n=1):
    return f"a{lo}" if n == 1 else f"a[{lo}:{lo + n - 1}]"


def vset(lo, n=1):
    return {("v", lo + i) for i in range(n)}


def aset(lo, n=1):
    return {("a", lo + i) for i in range(n)}


class Emitter:
    def __init__(self):
        self.out = []
        self.t = 0                 # wait states issued so far
        self.mfma_w = {}           # reg -> time of the MFMA that wrote it
        self.mfma_lat = {}         # reg -> wait states its MFMA result needs (12 where not listed)
        self.valu_w = {}
        self.trans_w = {}
        self.dot_w = {}
        self.c_read = {}           # reg -> time of the MFMA that read it as C without writing it
        self._skip = None
        self.lds_fifo = []         # outstanding LDS reads, oldest first: sets of dst regs
        self.lds_time = []         # ... and when each was issued
        self.wait_old = None       # a wait also covers younger reads issued at least this long ago
        self.stats = {"nop": 0, "wait": 0, "mfma": 0, "valu": 0, "lds": 0}
        self._m0_t = None

    def _raw(self, text, states=1):
        self.out.append(text)
        self.t += states

    def _need_gap(self, t_def, gap):
        between = self.t - t_def - 1
        if between < gap:
            n = gap - between
            self.stats["nop"] += n
            while n > 0:
                k = min(n, 16)
                self._raw(f"s_nop {k - 1}", k)
                n -= k

    def _wait_lds(self, regs):
        need = None
        for i, dst in enumerate(self.lds_fifo):
            if dst & regs:
                need = i
        if need is None:
            return
        if self.wait_old is not None:
            # younger reads that have very likely landed as well: waiting for them too costs nothing
            # now and saves the separate wait of their first use
            while need + 1 < len(self.lds_fifo) and self.lds_time[need + 1] <= self.t - self.wait_old:
                need += 1
        newer = len(self.lds_fifo) - 1 - need
        self.stats["wait"] += 1
        self._raw(f"s_waitcnt lgkmcnt({min(newer, 15)})")
        # everything up to `need` has returned (and more, if the count was clamped)
        done = max(need + 1, len(self.lds_fifo) - 15) if newer > 15 else need + 1
        self.lds_fifo = self.lds_fifo[done:]
        self.lds_time = self.lds_time[done:]

    def mfma(self, dst, a, b, c, dst_regs, a_regs, b_regs, c_regs):
        self._wait_lds(a_regs | b_regs | c_regs | dst_regs)
        for r in a_regs | b_regs:
            if r in self.mfma_w:
                self._need_gap(self.mfma_w[r], self.mfma_lat.get(r, 12))
        for r in c_regs - dst_regs:  # the result of another chain as accumulator input
            if r in self.mfma_w:
                self._need_gap(self.mfma_w[r], self.mfma_lat.get(r, 12))
        for r in a_regs | b_regs | c_regs:
            if r in self.valu_w:
                self._need_gap(self.valu_w[r], 2)
        for r in dst_regs - c_regs:  # overwriting without accumulating: order after VALU writers
            if r in self.valu_w:
                self._need_gap(self.valu_w[r], 2)
        self._raw(f"v_mfma_f32_32x32x16_bf16 {dst}, {a}, {b}, {c}")
        for r in c_regs - dst_regs:
            self.c_read[r] = self.t - 1
        for r in dst_regs:
            self.mfma_w[r] = self.t - 1
            self.mfma_lat.pop(r, None)
            self.valu_w.pop(r, None)
            self.trans_w.pop(r, None)
        self.stats["mfma"] += 1

    def mfma_f32x2(self, dst, a, b, dst_regs, a_regs, b_regs):
        """D[32 x 32] = A[32 x 2] B[2 x 32] in fp32 (16 passes, no accumulator input): one register of A
        (lane: row lane % 32, k = lane / 32) and one of B (k = lane / 32, column lane % 32)."""
        self._wait_lds(a_regs | b_regs | dst_regs)
        for r in a_regs | b_regs:
            if r in self.mfma_w:
                self._need_gap(self.mfma_w[r], self.mfma_lat.get(r, 12))
        for r in a_regs | b_regs | dst_regs:
            if r in self.valu_w:
                self._need_gap(self.valu_w[r], 2)
        self._raw(f"v_mfma_f32_32x32x2_f32 {dst}, {a}, {b}, 0")
        for r in dst_regs:
            self.mfma_w[r] = self.t - 1
            self.mfma_lat[r] = 20
            self.valu_w.pop(r, None)
            self.trans_w.pop(r, None)
        self.stats["mfma32"] = self.stats.get("mfma32", 0) + 1

    def valu(self, text, dst_regs, src_regs, trans=False):
        is_dot = text.startswith("v_dot2c")
        self._wait_lds(dst_regs | src_regs)
        for r in dst_regs | src_regs:
            if r in self.mfma_w:
                self._need_gap(self.mfma_w[r], self.mfma_lat.get(r, 12))
        for r in src_regs:
            if r in self.trans_w:
                self._need_gap(self.trans_w[r], 1)
        for r in dst_regs | src_regs:
            if r in self.dot_w and not (is_dot and r in dst_regs):
                self._need_gap(self.dot_w[r], 4)
        for r in dst_regs:
            if r in self.c_read:
                self._need_gap(self.c_read.pop(r), 12)
        self._raw(text)
        for r in dst_regs:
            self.mfma_w.pop(r, None)
            self.valu_w[r] = self.t - 1
            if trans:
                self.trans_w[r] = self.t - 1
            else:
                self.trans_w.pop(r, None)
            if is_dot:
                self.dot_w[r] = self.t - 1
            else:
                self.dot_w.pop(r, None)
        self.stats["valu"] += 1

    def lds_read(self, text, dst_regs):
        self._wait_lds(dst_regs)  # an older read into the same registers must have landed
        for r in dst_regs:
            if r in self.mfma_w:
                self._need_gap(self.mfma_w[r], self.mfma_lat.get(r, 12))
            if r in self.c_read:
                self._need_gap(self.c_read.pop(r), 12)
            self.mfma_w.pop(r, None)
            self.valu_w.pop(r, None)
            self.trans_w.pop(r, None)
        self._raw(text)
        self.lds_fifo.append(set(dst_regs))
        self.lds_time.append(self.t - 1)
        self.stats["lds"] += 1

    def lds_direct_load(self, lds_imm, goff, gbase, ldsn="%[ldsn]"):
        """Next step's global -> LDS copy of one 1 KB block (M0 = LDS destination)."""
        self.lds_direct_dest(lds_imm, ldsn)
        self.lds_direct_issue(goff, gbase)

    def lds_direct_dest(self, lds_imm, ldsn="%[ldsn]"):
        """M0 for the next LDS-direct load.  The load needs one wait state after the write: callers
        that put other instructions in between save the s_nop."""
        self._raw(f"s_add_u32 m0, {ldsn}, {lds_imm}")
        self._m0_t = self.t - 1

    def lds_direct_issue(self, goff, gbase):
        self._need_gap(self._m0_t, 1)
        self._raw(f"global_load_lds_dwordx4 {goff}, {gbase}")
        self.stats["vmem"] = self.stats.get("vmem", 0) + 1

    def lds_direct_load_chained(self, goff, gbase, next_imm, ldsn="%[ldsn]"):
        """An LDS-direct load whose M0 was written behind the previous one (the first one's by the code in
        front of the stream), followed by the M0 write of the next one: no wait state is spent between the
        write and its load."""
        if getattr(self, "_m0_t", None) is None:
            self._m0_t = -(1 << 20)   # written before the stream
        self.lds_direct_issue(goff, gbase)
        if next_imm is not None:
            self.lds_direct_dest(next_imm, ldsn)

    def vmem_store(self, text, src_regs):
        """A store to global memory from VGPRs (it joins the in-order vector-memory queue)."""
        self._wait_lds(src_regs)
        for r in src_regs:
            if r in self.mfma_w:
                self._need_gap(self.mfma_w[r], self.mfma_lat.get(r, 12))
        self._raw(text)
        self.stats["vmem"] = self.stats.get("vmem", 0) + 1

    def lds_write(self, text, src_regs):
        """An LDS store: takes a place in the in-order LDS queue like a read."""
        self._wait_lds(src_regs)
        for r in src_regs:
            if r in self.mfma_w:
                self._need_gap(self.mfma_w[r], self.mfma_lat.get(r, 12))
        self._raw(text)
        self.lds_fifo.append(set())
        self.lds_time.append(self.t - 1)
        self.stats["lds"] += 1

    def raw(self, text):
        """Scalar or wait instruction with no tracked vector registers."""
        self._raw(text)

    def label(self, text):
        self._raw(text, 0)

    _TRACKED = ("mfma_w", "valu_w", "trans_w", "dot_w", "c_read")  # (mfma_lat only grows entries for live mfma_w ones)

    def skip_begin(self):
        """The instructions up to skip_end() may be jumped over by the branch emitted just before."""
        assert self._skip is None
        self._skip = (self.t, {n: dict(getattr(self, n)) for n in self._TRACKED}, len(self.lds_fifo))

    def skip_end(self):
        t0, saved, n_lds = self._skip
        self._skip = None
        assert len(self.lds_fifo) == n_lds, "no LDS operations inside a skippable block"
        for n in self._TRACKED:
            merged = dict(saved[n])
            for r, t in getattr(self, n).items():
                merged[r] = max(merged.get(r, -1 << 30), min(t, t0 - 1))
            setattr(self, n, merged)
        self.t = t0

    def drain(self):
        if self.lds_fifo:
            self._raw("s_waitcnt lgkmcnt(0)")
            self.lds_fifo = []
            self.lds_time = []


class Op:
    """A unit the scheduler places as a whole: `emit(em)` writes it; `cost` is its share of an MFMA
    gap; it goes into gap `earliest` at the soonest and must be out before MFMA number `deadline`."""

    def __init__(self, emit, cost=1, earliest=0, deadline=None):
        self.emit, self.cost, self.earliest, self.deadline = emit, cost, earliest, deadline


def address_flips(reads, make_op, pattern=r"%\[([rt]\d)\]"):
    """Chain of operations that flip the LDS operand addresses between the two step buffers (XOR with
    0x10000), each placed behind the last read of the step that uses the address: in the stream they hide
    in the gaps between MFMAs, behind the loop's barrier nothing hides them.  `reads`: (text, deadline) of
    every LDS read of the step; `make_op(name, earliest)` builds the flip of operand `name`."""
    import re
    last = {}
    for text, deadline in reads:
        for name in re.findall(pattern, text):
            last[name] = max(last.get(name, 0), deadline)
    return [make_op(name, at + 1) for name, at in sorted(last.items(), key=lambda kv: kv[1])]


def schedule(em, mfmas, chains, cap):
    """Writes the MFMAs in order with the chains' operations in the gaps between them (gap g lies in
    front of MFMA g; gap len(mfmas) behind the last one).  A single wave only keeps the matrix pipe
    busy while the instructions between two MFMAs issue within the 32 cycles the first one runs, about
    four of them: so every gap takes at most `cap` units of cost unless deadlines force more, picked
    earliest-deadline-first among the chains' heads (order inside a chain is kept)."""
    n = len(mfmas)
    big = 1 << 30
    for ch in chains:  # an operation inherits the needs of its neighbours in the chain
        e = 0
        for op in ch:
            e = op.earliest = max(op.earliest, e)
        d = big
        for op in reversed(ch):
            d = op.deadline = min(big if op.deadline is None else op.deadline, d)
            assert op.earliest <= op.deadline, "an operation's window is empty"
    heads = [0] * len(chains)
    over = 0
    for g in range(n + 1):
        used = 0
        while True:
            best = None
            for i, ch in enumerate(chains):
                if heads[i] < len(ch):
                    op = ch[heads[i]]
                    if op.earliest <= g and (best is None or op.deadline < chains[best][heads[best]].deadline):
                        best = i
            if best is None:
                break
            op = chains[best][heads[best]]
            forced = op.deadline <= g or g == n
            if not forced and used + op.cost > cap:
                break
            op.emit(em)
            used += op.cost
            heads[best] += 1
        over += max(0, used - cap)
        if g < n:
            if callable(mfmas[g]):
                mfmas[g](em)
            else:
                em.mfma(*mfmas[g])
    assert all(heads[i] == len(ch) for i, ch in enumerate(chains)), "operations left over"
    em.stats["over_cap"] = over

