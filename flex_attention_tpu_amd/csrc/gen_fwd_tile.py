#!/usr/bin/env python3
"""Generator of the hand-scheduled gfx950 instruction streams of the bf16 forward kernel (plain
score).  Writes fwd_tile.inc: string-literal macros that fwd_bf16.hip places inside `asm volatile`
statements: the run loop over steps of two 64-row kv tiles, and prologue / epilogue register moves.

A wave owns 2 x 32 q rows (q blocks x = 0, 1): their Q^T fragments and O^T accumulators stay in
accumulation registers, so every K / V fragment read from LDS feeds two MFMAs.  One step covers
128 kv rows = four 32-row kv blocks c = 0..3, software-pipelined:

    A(c): S'^T = K Q^T - M for both q blocks   16 MFMAs, operands: 8 ds_read_b128 (rows of K)
    E(c, x): online softmax of the lane's 16 scores of q block x (45 VALU ops)
    B(c, x): O^T += V^T P^T of q block x       8 MFMAs, operands: 32 ds_read_b64_tr_b16 (V), read once
             for both q blocks

    The two q blocks run half a stage apart: E(c, 0) under A(c+1)[k-steps 0-3] and B(c-1, 1),
    E(c, 1) under A(c+1)[k-steps 4-7] and B(c, 0).

The softmax is arranged so that the common case costs no arithmetic beyond exp, pack and sum:
  * Q arrives pre-multiplied by sm_scale * log2(e), so the MFMA result is already in the log2 domain;
  * the reference maximum M the probabilities are taken against, p = 2^(t - M), enters through the
    accumulator input of the first MFMA of each chain (16 registers per q block hold -M), so the
    chain's result is t - M and p is a bare v_exp_f32;
  * M only moves when the running maximum relative to it, Mt = max(t - M), leaves [-TAU, TAU] (p then
    stays inside 2^+-TAU: safe for bf16 and fp32).  The move is a skipped-unless-needed block right
    behind the test: O^T, L, the block's scores and the -M registers are corrected by the lane's
    shift, and the chain of the next kv block, already in flight with the old -M, is corrected by a
    second such block at the start of its own softmax;
  * the row sum L accumulates the fp32 p.
State per q row: M, Mt (true maximum = M + Mt), L.  The C++ epilogue turns them into the exact
(m, l) outputs.

Register contract with the C++ side (every asm statement names the accumulation registers with
physical-register constraints):
    a[0:63], a[64:127]     O^T accumulators of q block 0, 1 (4 x 16 each)
    a[128:159], a[160:191] Q^T fragments of q block 0, 1 (8 x 4 each), pre-scaled
    a[192:255]             staging slots of the LDS fragments (clobbered)
    v[66:199], s[60:100], vcc, m0   scratch of the run loop (clobbered)
    %[r0..r7]  byte address of the lane's row fragment ks in K half-tile 0 of the current buffer
    %[t0..t7]  byte address of the lane's transposed fragment (2 db + hi) in K half-tile 0 (the V
               tiles lie 32 KiB behind the K tiles)
    %[M0], %[M1], %[Mt0], %[Mt1], %[L0], %[L1]  softmax state of the lane's two q rows (in/out);
               start values 0, -inf, 0
    %[g0], %[g1v], %[g2], %[g3]  the lane's byte offsets inside a global half tile for the wave's 1 KB blocks
    %[m0] .. %[m3]  (partial steps) keep bits of q block x, kv tile h in m[2 x + h]: bit 16 (c & 1) + e is
               element e of kv block c (c >> 1 == h); dropped elements get score -inf
    %[tbl]     LDS byte address of the wave's table of work-group constants (TABLE below)
    %[lst]     LDS byte address of the item's merged kv tile list (int32 entries)
    %[it], %[kba1], %[kbb1], %[buf]  loop state (in/out); %[it_end], %[partial]  (in)
LDS layout of one step buffer (bytes): K tile 0, K tile 1, V tile 0, V tile 1 (16 KiB each); the two
buffers are 64 KiB apart and the first starts at LDS address 0.
"""
import argparse
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from gfx950_stream import Emitter, Op, address_flips, ar, aset, schedule, vr, vset  # noqa: E402

MIN_AHEAD = 2    # MFMA pairs at least between the LDS reads of a pair and its MFMAs
WAIT_OLD = 20    # a wait for LDS data also covers younger reads issued at least this many instructions ago
CAP = 6          # instructions the scheduler puts between two MFMAs unless deadlines force more
LOAD_FIRST = 2   # MFMA gap from which the first LDS-direct load of the next step may go out
LOAD_EVERY = 2   # gaps between two of them
LOAD_COST = 3    # share of an MFMA gap one of them takes
TAU = "0x40c00000"  # 6.0: M moves when the running maximum relative to it leaves [-6, 6]
TRANS_COST = 2   # share of an MFMA gap a transcendental takes (it holds the wave's issue for two slots)
ROUNDED_SUM = False  # row sums add the bf16-rounded probabilities (v_dot2c on the packed pairs) instead of the fp32 ones
DROP = ()        # instruction classes left out (--drop, timing studies only)
CAP_SOFTCAP = 8  # instructions per MFMA gap in the softcap variant (6.5 VALU ops per score instead of 2.5)
S_K2 = "s62"     # (softcap variant) -2 cap log2(e): the table's c2 entry
SEQUENTIAL = True  # (plain scores) the S chains of the two q blocks one after the other instead of alternating

TILE = 16384
# No scalar operands: constants come from a per-wave table in LDS, loop state from VGPR operands.
TABLE = ["n_list", "w4k", "c2", "n_steps", "kg_lo", "kg_hi", "vg_lo", "vg_hi", "kban", "kbbn", "kgn_lo", "kgn_hi",
         "vgn_lo", "vgn_hi", "pad0", "pad1"]
SREG = {"n_list": "s60", "w4k": "s61", "c2": "s62", "n_steps": "s63", "kg_lo": "s64", "kg_hi": "s65", "vg_lo": "s66",
        "vg_hi": "s67", "kban": "s68", "kbbn": "s69", "kgn_lo": "s70", "kgn_hi": "s71", "vgn_lo": "s78", "vgn_hi": "s79",
        "pad0": "s80", "pad1": "s81",
        "it": "s72", "kba1": "s73", "kbb1": "s74", "buf": "s75", "it_end": "s76", "partial": "s77"}
STATE_IO = ["it", "kba1", "kbb1", "buf"]
STATE_IN = ["it_end", "partial"]
S_T = ["s84", "s85", "s86", "s87"]   # temporaries of the loop top / tail; s[86:87] also inside the masked stream
S_GK0, S_GK1, S_GV0, S_GV1 = "s[88:89]", "s[90:91]", "s[92:93]", "s[94:95]"
S_SEL = ["s82", "s83", "s96", "s97", "s98", "s99"]
S_LDSN = "s100"
S_PEND = ["s80", "s81"]   # per q block: the chain in flight still carries the old -M (reuses the pad slots)
V_KB2 = 66       # 2 temporaries of the loop tail
V_MSK = 68       # 4 temporaries of the masked variant
V_TBL = 72       # 16 scratch VGPRs the table is read into at entry
V_S0 = 72        # S^T accumulators [c & 1][x] x 16
V_P0 = 136       # P^T as MFMA B operands [x][u] x 4 (B(c, x) has issued before E(c + 1, x) writes again)
V_NEGM = 152     # -M of q block 0, 1, 16 copies each: accumulator input of a chain's first MFMA
V_TMP = 184      # 10 temporaries of the softmax
V_NEGINF = 194
V_TAU = 195
V_D = 196        # shift of M of q block 0, 1 (0 in lanes that keep theirs)
V_AL = 198       # 2^-shift of q block 0, 1
V_END = 199
A_O, A_Q, A_STG = 0, 128, 192
# Position-bias variant (score + slope (j - i)): the accumulator input of the S chain of kv block c, q block
# x, slope' (j - i) - M with slope' = slope log2(e), is itself a matrix product, [1, r] x [b; slope'] with r the
# key's row in the block and b = slope' (j0 - i) - M for the block's first key j0: one fp32 MFMA per
# chain writes it into the registers that hold -M in the plain variant.
#   %[aone]  A operand: 1.0 in lanes 0-31, float(lane - 32) in lanes 32-63
#   %[mulv]  slope' in lanes 0-31, 0 in lanes 32-63
#   %[addv0], %[addv1]  -M of the lane's q row resp. slope' (in/out: they follow M)
#   %[iq]    the lane's q index in q block 0 (q block 1: 128 more);  %[ka0], %[kb0]  kv tiles of the run's first step
# The kv list is walked from its end: with a positive slope the bias grows with the key index, so the
# running maximum settles in the first steps instead of moving the reference M at every block.
V_B = [200, 201]   # B operands (alternating)
V_T = V_TMP + 9
V_END_ALIBI = 201
S_CUR = ["s62", "s101"]  # kv tiles of the current step


def bias_ops(e, c, q, tile):
    """The accumulator input of the S chain (c, q): keys from 64 `tile` + 32 (c & 1) on, q rows 128 q on."""
    t0 = S_T[0]
    b = V_B[q]
    off = 32 * (c & 1) - 128 * q
    e.raw(f"s_lshl_b32 {t0}, {tile}, 6")
    if off > 0:
        e.raw(f"s_add_u32 {t0}, {t0}, {off}")
    elif off < 0:
        e.raw(f"s_sub_u32 {t0}, {t0}, {-off}")
    e.valu(f"v_sub_u32_e32 {vr(V_T)}, {t0}, %[iq]", vset(V_T), set())
    e.valu(f"v_cvt_f32_i32_e32 {vr(V_T)}, {vr(V_T)}", vset(V_T), vset(V_T))
    e.valu(f"v_fma_f32 {vr(b)}, %[mulv], {vr(V_T)}, %[addv{q}]", vset(b), vset(V_T) | {("op", f"addv{q}")})
    e.mfma_f32x2(vr(V_NEGM + 16 * q, 16), "%[aone]", vr(b), vset(V_NEGM + 16 * q, 16), set(), vset(b))


def v_s(c, x):
    return V_S0 + 32 * (c & 1) + 16 * x


def v_p(c, x, u):
    return V_P0 + 8 * x + 4 * u


def build(masked, alibi=False, softcap=False):
    em = Emitter()
    em.wait_old = WAIT_OLD
    # MFMA pairs (2 MFMAs each), in issue order.  The two q blocks of a kv block are processed half a
    # stage apart: E(c, 0) runs under A(c+1)[ks 0-3] and B(c-1, 1), E(c, 1) under A(c+1)[ks 4-7] and
    # B(c, 0), so every softmax has MFMAs of both kinds to hide under.
    pairs = []

    def add_A(c, lo, hi):
        for ks in range(lo, hi):
            pairs.append(("A", c, ks))

    def add_B(c, q):
        for u in range(2):
            for j in range(2):
                pairs.append(("B", c, (q, u, j)))

    # Without a position bias the S chains of the two q blocks run one after the other (a chain's eight
    # MFMAs issue back to back at full rate): the first chain of a kv block is finished eight MFMAs earlier
    # than when the two alternate, its softmax starts that much earlier, and the softmax work spreads over
    # the step instead of crowding behind A(0).  A pair is then two k-steps of one chain.
    sequential = SEQUENTIAL and not alibi

    def add_S(c, q):
        for j in range(4):
            pairs.append(("A", c, (q, j)))

    if sequential:
        for kind, c, q in (("S", 0, 0), ("S", 0, 1), ("S", 1, 0), ("B", 0, 0), ("S", 1, 1), ("B", 0, 1), ("S", 2, 0), ("B", 1, 0),
                           ("S", 2, 1), ("B", 1, 1), ("S", 3, 0), ("B", 2, 0), ("S", 3, 1), ("B", 2, 1), ("B", 3, 0), ("B", 3, 1)):
            (add_S if kind == "S" else add_B)(c, q)
    else:
        add_A(0, 0, 8)
        for c in range(4):
            for q in range(2):
                if c < 3:
                    add_A(c + 1, 4 * q, 4 * q + 4)
                if q == 1:
                    add_B(c, 0)
                elif c > 0:
                    add_B(c - 1, 1)
        add_B(3, 1)
    idx = {key: 2 * k for k, key in enumerate(pairs)}  # number of the pair's first MFMA
    n_mfma = 2 * len(pairs)

    def a_mfma(c, ks, q):     # S chain of q block q: MFMA number of k-step ks
        if sequential:
            return idx[("A", c, (q, ks >> 1))] + (ks & 1)
        return idx[("A", c, ks)] + q

    def b_first(c, q, u):
        return idx[("B", c, (q, u, 0))]

    def b_last(c, q, u):
        return idx[("B", c, (q, u, 1))] + 1

    def half_off(c):
        return (c >> 1) * TILE + (c & 1) * (TILE // 2)

    # Staging registers.  K row fragments rotate through eight 4-register slots.  The V^T fragments of
    # a kv block have fixed places: B(c, 0) loads them, B(c, 1) half a stage later uses them again,
    # and the fragments of block c + 1 are read in once the MFMA of B(c, 1) that used the place has
    # been issued.
    a_index = {}
    for k, (kind, c, x) in enumerate(pairs):
        if kind == "A":
            a_index[k] = len(a_index)
    a_pairs = [k for k in range(len(pairs)) if pairs[k][0] == "A"]

    def k_slot(k):
        return A_STG + 32 + 4 * (a_index[k] % 8)

    def ks_slot(ks):          # (sequential chains: the fragment of k-step ks has its own slot, read once for both chains)
        return A_STG + 32 + 4 * ks

    def v_place(u, db):
        return A_STG + 4 * (4 * u + db)

    holds = {}  # V^T place -> kv block whose fragment was last read into it

    def valu(text, dst, src, trans=False, **kw):
        return Op((lambda e: e.valu(text, dst, src, trans)) if "valu" not in DROP else (lambda e: None),
                  cost=TRANS_COST if trans else 1, **kw)

    reads = []
    read_texts = []
    for k, (kind, c, x) in enumerate(pairs):
        if kind == "A" and sequential:
            q, j = x
            for ks in (2 * j, 2 * j + 1) if q == 0 else ():
                text, dst = f"ds_read_b128 {ar(ks_slot(ks), 4)}, %[r{ks}] offset:{half_off(c)}", aset(ks_slot(ks), 4)
                earliest = a_mfma(c - 1, ks, 1) + 1 if c > 0 else 0   # (the slot's last user: the second chain of block c - 1)
                reads.append((2 * k, Op((lambda e, t=text, d=dst: e.lds_read(t, d)) if "lds" not in DROP else (lambda e: None),
                                        earliest=earliest, deadline=max(0, 2 * (k - MIN_AHEAD)))))
                read_texts.append((text, max(0, 2 * (k - MIN_AHEAD))))
        elif kind == "A":
            ia = a_index[k]
            text, dst = f"ds_read_b128 {ar(k_slot(k), 4)}, %[r{x}] offset:{half_off(c)}", aset(k_slot(k), 4)
            earliest = 2 * a_pairs[ia - 8] + 2 if ia >= 8 else 0
            reads.append((2 * k, Op((lambda e, t=text, d=dst: e.lds_read(t, d)) if "lds" not in DROP else (lambda e: None),
                                    earliest=earliest, deadline=max(0, 2 * (k - MIN_AHEAD)))))
            read_texts.append((text, max(0, 2 * (k - MIN_AHEAD))))
        elif x[0] == 0:
            q, u, j = x
            off = 2 * TILE + half_off(c) + u * 4096
            for db in (2 * j, 2 * j + 1):
                for hi in range(2):
                    reg = v_place(u, db) + 2 * hi
                    text, dst = f"ds_read_b64_tr_b16 {ar(reg, 2)}, %[t{2 * db + hi}] offset:{off}", aset(reg, 2)

                    def emit(e, t=text, d=dst, key=(u, db), blk=c):
                        holds[key] = blk
                        if "lds" not in DROP:
                            e.lds_read(t, d)
                    earliest = b_last(c - 1, 1, u) + 1 if c > 0 else 0
                    reads.append((2 * k, Op(emit, earliest=earliest, deadline=2 * (k - MIN_AHEAD))))
                    read_texts.append((text, 2 * (k - MIN_AHEAD)))
    reads.sort(key=lambda r: r[0])  # (stable: in the order of their use)

    def mfma_of(k, j):
        kind, c, x = pairs[k]
        if kind == "A":
            if sequential:
                q, ks = x[0], 2 * x[1] + j
                slot = ks_slot(ks)
            else:
                ks, q = x, j
                slot = k_slot(k)
            s = v_s(c, q)
            # the chain starts from -M: its result is the score relative to the reference maximum
            cin = V_NEGM + 16 * q if ks == 0 else s
            if softcap and ks == 0:   # (softcap: the result is the exponent of e^(2 s / cap), nothing to start from)
                return (vr(s, 16), ar(slot, 4), ar(A_Q + 32 * q + 4 * ks, 4), "0", vset(s, 16), aset(slot, 4),
                        aset(A_Q + 32 * q + 4 * ks, 4), set())
            return (vr(s, 16), ar(slot, 4), ar(A_Q + 32 * q + 4 * ks, 4), vr(cin, 16), vset(s, 16), aset(slot, 4),
                    aset(A_Q + 32 * q + 4 * ks, 4), vset(cin, 16))
        q, u, jj = x
        db = 2 * jj + j
        p = v_p(c, q, u)
        acc = A_O + 64 * q + 16 * db
        vt = v_place(u, db)
        args = (ar(acc, 16), ar(vt, 4), vr(p, 4), ar(acc, 16), aset(acc, 16), aset(vt, 4), vset(p, 4), aset(acc, 16))

        def emit(e):
            assert holds.get((u, db)) == c, f"B({c}, {q}) would multiply with the V^T fragment of block {holds.get((u, db))}"
            e.mfma(*args)
        return emit

    mfmas = [mfma_of(k, j) for k in range(len(pairs)) for j in range(2)]
    if "mfma" in DROP:
        mfmas = [(lambda e: None)] * n_mfma

    # ---- VALU work of E(c, q) -------------------------------------------------------------------
    T = [V_TMP + i for i in range(10)]
    tag = "m" if masked else "f"

    def block(ops, **kw):
        """A branch, the block it may skip and its label, placed as one unit."""
        def emit(e):
            for op in ops:
                if op[0] == "raw":
                    e.raw(op[1])
                elif op[0] == "label":
                    e.label(op[1])
                elif op[0] == "skip_begin":
                    e.skip_begin()
                elif op[0] == "skip_end":
                    e.skip_end()
                elif "valu" not in DROP:
                    e.valu(*op[1:])
        return Op(emit, cost=2, **kw)

    late_sums = []

    def softmax_chain(c, q):
        """Online softmax of the lane's 16 scores (relative to M) of q block q in kv block c."""
        s = v_s(c, q)
        M, Mt, L = f"%[M{q}]", f"%[Mt{q}]", f"%[L{q}]"
        kM, kMt, kL = {("op", f"M{q}")}, {("op", f"Mt{q}")}, {("op", f"L{q}")}
        D, AL, negm = V_D + q, V_AL + q, V_NEGM + 16 * q
        ops = []

        if softcap:
            # Scores are bounded by the cap, so the reference maximum is the constant cap and nothing is tracked:
            # the chain gave u with e^(2 s / cap) = 2^u; r = 1 / (2^u + 1), tanh = 1 - 2 r, and
            # p = 2^(cap' tanh - cap') = 2^(-2 cap' r) with cap' = cap log2(e) (S_K2 holds -2 cap').
            def packs_sc(g):
                u2 = g >> 1
                war = b_last(c - 1, q, u2) + 1 if c > 0 else 0   # the registers are those of block c - 1
                for h in range(2):
                    e = 4 * g + 2 * h
                    pr = v_p(c, q, u2) + 2 * (g & 1) + h
                    ops.append(valu(f"v_cvt_pk_bf16_f32 {vr(pr)}, {vr(s + e)}, {vr(s + e + 1)}", vset(pr), vset(s + e, 2),
                                    earliest=war, deadline=b_first(c, q, u2) - 1))
            for g in range(4):
                for text, trans in (("v_exp_f32_e32 {s}, {s}", True), ("v_add_f32_e32 {s}, 1.0, {s}", False),
                                    ("v_rcp_f32_e32 {s}, {s}", True), (f"v_mul_f32_e32 {{s}}, {S_K2}, {{s}}", False),
                                    ("v_exp_f32_e32 {s}, {s}", True)):
                    for u in range(4):
                        e = 4 * g + u
                        ops.append(valu(text.format(s=vr(s + e)), vset(s + e), vset(s + e), trans))
                if masked:
                    for u in range(4):
                        e = 4 * g + u
                        ops.append(valu(f"v_bfe_i32 {vr(V_MSK + u)}, %[m{2 * q + (c >> 1)}], {16 * (c & 1) + e}, 1", vset(V_MSK + u), set()))
                    for u in range(4):
                        e = 4 * g + u   # keep ? p : 0
                        ops.append(valu(f"v_and_b32_e32 {vr(s + e)}, {vr(s + e)}, {vr(V_MSK + u)}", vset(s + e), vset(s + e) | vset(V_MSK + u)))
                packs_sc(g)
                for u in range(4):
                    e = 4 * g + u
                    ops.append(valu(f"v_add_f32_e32 {L}, {L}, {vr(s + e)}", kL, kL | vset(s + e)))
            ops[0].earliest = max(ops[0].earliest, a_mfma(c, 7, q) + 4)   # the chain's last result needs 12 wait states
            if c + 2 < 4:
                ops[-1].deadline = min(ops[-1].deadline or (1 << 30), a_mfma(c + 2, 0, q))  # A(c + 2) writes the same S registers
            return ops

        if c > 0 and not sequential:
            # M moved while this block's chain was in flight with the old -M: apply the shift now
            late = [("raw", f"s_cmp_eq_u32 {S_PEND[q]}, 0"), ("raw", f"s_cbranch_scc1 .Lfa_fwd_{tag}_late{c}{q}_%="), ("skip_begin",)]
            for e in range(16):
                late.append(("valu", f"v_sub_f32_e32 {vr(s + e)}, {vr(s + e)}, {vr(D)}", vset(s + e), vset(s + e) | vset(D), False))
            late += [("raw", f"s_mov_b32 {S_PEND[q]}, 0"), ("skip_end",), ("label", f".Lfa_fwd_{tag}_late{c}{q}_%=:")]
            ops.append(block(late))
        if masked:
            for g in range(4):
                for u in range(4):
                    e = 4 * g + u
                    ops.append(valu(f"v_bfe_i32 {vr(V_MSK + u)}, %[m{2 * q + (c >> 1)}], {16 * (c & 1) + e}, 1", vset(V_MSK + u), set()))
                for u in range(4):
                    e = 4 * g + u  # keep ? score : -inf
                    ops.append(valu(f"v_bfi_b32 {vr(s + e)}, {vr(V_MSK + u)}, {vr(s + e)}, {vr(V_NEGINF)}", vset(s + e),
                                    vset(s + e) | vset(V_MSK + u) | vset(V_NEGINF)))
        # block maximum of the lane's 16 scores, then across the two half-waves that share the q row
        for i in range(5):
            ops.append(valu(f"v_max3_f32 {vr(T[i])}, {vr(s + 3 * i)}, {vr(s + 3 * i + 1)}, {vr(s + 3 * i + 2)}", vset(T[i]), vset(s + 3 * i, 3)))
        ops.append(valu(f"v_max3_f32 {vr(T[0])}, {vr(T[0])}, {vr(T[1])}, {vr(T[2])}", vset(T[0]), vset(T[0]) | vset(T[1]) | vset(T[2])))
        ops.append(valu(f"v_max3_f32 {vr(T[3])}, {vr(T[3])}, {vr(T[4])}, {vr(s + 15)}", vset(T[3]), vset(T[3]) | vset(T[4]) | vset(s + 15)))
        ops.append(valu(f"v_max_f32_e32 {vr(T[0])}, {vr(T[0])}, {vr(T[3])}", vset(T[0]), vset(T[0]) | vset(T[3])))
        # Mt is the running maximum of the lane's own 16 of the row's 32 scores per block (the two half-waves
        # that share a q row meet in the block below and in the kernel's epilogue): the common path needs no
        # exchange between lanes.
        ops.append(valu(f"v_max_f32_e32 {Mt}, {Mt}, {vr(T[0])}", kMt, kMt | vset(T[0])))

        # does a running maximum leave [-TAU, TAU] (and is it finite: lanes that kept nothing so far stay put)?
        def leaves():
            t = [("valu", f"v_cmp_gt_f32_e64 vcc, |{Mt}|, {vr(V_TAU)}", set(), kMt | vset(V_TAU), False)]
            if masked:
                t.append(("valu", f"v_cmp_neq_f32_e64 s[86:87], {Mt}, {vr(V_NEGINF)}", set(), kMt | vset(V_NEGINF), False))
                t.append(("raw", "s_and_b64 vcc, vcc, s[86:87]"))
            return t
        rare = leaves()
        rare += [("raw", f"s_cbranch_vccz .Lfa_fwd_{tag}_keep{c}{q}_%="), ("skip_begin",), ("raw", "s_nop 3"),
                 # some lane's maximum left the band: the row's maximum into both of its lanes, then the test
                 # again, now the same for both (a lane whose half of the keys lags behind the other's gets
                 # here once and carries the row's maximum from then on)
                 ("valu", f"v_mov_b32_e32 {vr(T[0])}, {Mt}", vset(T[0]), kMt, False),
                 ("valu", f"v_mov_b32_e32 {vr(T[1])}, {Mt}", vset(T[1]), kMt, False),
                 ("raw", "s_nop 1"),
                 ("valu", f"v_permlane32_swap_b32 {vr(T[0])}, {vr(T[1])}", vset(T[0]) | vset(T[1]), vset(T[0]) | vset(T[1]), False),
                 ("raw", "s_nop 1"),
                 ("valu", f"v_max_f32_e32 {Mt}, {vr(T[0])}, {vr(T[1])}", kMt, vset(T[0]) | vset(T[1]), False)]
        rare += leaves() + [("raw", "s_nop 3"),
                 ("valu", f"v_cndmask_b32_e32 {vr(D)}, 0, {Mt}, vcc", vset(D), kMt, False),                 # the lane's shift
                 # (2^-shift, the shift held above -126: what was summed against a reference more than 2^126 too
                 # high has been flushed to zero and must stay zero, not become 0 x inf)
                 ("valu", f"v_max_f32_e32 {vr(AL)}, 0xc2fc0000, {vr(D)}", vset(AL), vset(D), False),
                 ("valu", f"v_exp_f32_e64 {vr(AL)}, -{vr(AL)}", vset(AL), vset(AL), True),
                 ("valu", f"v_sub_f32_e32 {Mt}, {Mt}, {vr(D)}", kMt, kMt | vset(D), False),
                 ("valu", f"v_add_f32_e32 {M}, {M}, {vr(D)}", kM, kM | vset(D), False),
                 ("valu", f"v_mul_f32_e32 {L}, {L}, {vr(AL)}", kL, kL | vset(AL), False)]
        for i in range(64):
            t = T[5 + (i % 4)]
            acc = A_O + 64 * q + i
            rare.append(("valu", f"v_accvgpr_read_b32 {vr(t)}, {ar(acc)}", vset(t), aset(acc), False))
            rare.append(("valu", f"v_mul_f32_e32 {vr(t)}, {vr(t)}, {vr(AL)}", vset(t), vset(t) | vset(AL), False))
            rare.append(("valu", f"v_accvgpr_write_b32 {ar(acc)}, {vr(t)}", aset(acc), vset(t), False))
        for e in range(16):
            rare.append(("valu", f"v_sub_f32_e32 {vr(s + e)}, {vr(s + e)}, {vr(D)}", vset(s + e), vset(s + e) | vset(D), False))
        for e in range(16):
            rare.append(("valu", f"v_sub_f32_e32 {vr(negm + e)}, {vr(negm + e)}, {vr(D)}", vset(negm + e), vset(negm + e) | vset(D), False))
        if alibi:
            # -M in lanes 0-31 of the B operand's source follows M (lanes 32-63 hold the slope)
            kA = {("op", f"addv{q}")}
            rare += [("raw", "s_mov_b32 s86, -1"), ("raw", "s_mov_b32 s87, 0"),
                     ("valu", f"v_cndmask_b32_e64 {vr(T[5])}, 0, {vr(D)}, s[86:87]", vset(T[5]), vset(D), False),
                     ("valu", f"v_sub_f32_e32 %[addv{q}], %[addv{q}], {vr(T[5])}", kA, kA | vset(T[5]), False)]
        if c < 3 and not sequential:
            rare.append(("raw", f"s_mov_b32 {S_PEND[q]}, 1"))  # (kv block c + 1 of this step is in flight; block 0 of the next step is not)
        rare += [("skip_end",), ("label", f".Lfa_fwd_{tag}_keep{c}{q}_%=:")]
        # The block rescales O^T: every B(c - 1, q) MFMA is out, no B(c, q) MFMA is; and the chain of
        # kv block c + 1 has started (it carries the old -M and is corrected by its own "late" block).
        rare_earliest = 0
        rare_deadline = None
        if c > 0:
            rare_earliest = b_last(c - 1, q, 1) + 1
        if c < 3 and sequential:
            # (sequential chains: the chain of kv block c + 1 starts behind this block and takes the corrected
            # -M registers as they are; nothing is ever in flight with the old ones)
            rare_deadline = a_mfma(c + 1, 0, q) - 1
        elif c < 3:
            rare_earliest = max(rare_earliest, a_mfma(c + 1, 0, q) + 1)
        if alibi and c < 3:
            # The accumulator input of chain (c + 2, q) (block 0 of the next step for c = 2) right in front
            # of the block that moves M, which corrects it like the plain -M: chain (c + 1, q), which read
            # the registers, is out by then; 20 wait states before the chain's first MFMA.
            cn = c + 2
            tile = S_CUR[1] if cn < 4 else S_SEL[0]
            ops.append(Op(lambda e: bias_ops(e, cn & 3, q, tile), cost=CAP, earliest=rare_earliest,
                          deadline=a_mfma(cn, 0, q) - 6 if cn < 4 else None))
        ops.append(block(rare, earliest=rare_earliest, deadline=rare_deadline))

        # p = 2^(score - M), packed to bf16 B operands.  The row sum adds the fp32 values: l is then the
        # softmax denominator of the logits themselves, which is what the backward kernels divide their
        # recomputed probabilities by.  (Summing the rounded values, v_dot2c on the packed pairs, makes
        # o = sum(p v) / sum(p) a convex combination whatever the rounding, but moves l, and with it every
        # probability of the row in the backward, by up to 2^-8 relative where a row has few dominant keys:
        # measured, that was the largest single share of the error of dk and dv.)
        def exps(g):
            for u in range(4):
                e = 4 * g + u
                ops.append(valu(f"v_exp_f32_e32 {vr(s + e)}, {vr(s + e)}", vset(s + e), vset(s + e), True))

        def packs(g):
            u2 = g >> 1
            war = b_last(c - 1, q, u2) + 1 if c > 0 else 0   # the registers are those of block c - 1
            for h in range(2):
                e = 4 * g + 2 * h
                pr = v_p(c, q, u2) + 2 * (g & 1) + h
                ops.append(valu(f"v_cvt_pk_bf16_f32 {vr(pr)}, {vr(s + e)}, {vr(s + e + 1)}", vset(pr), vset(s + e, 2),
                                earliest=war, deadline=b_first(c, q, u2) - 1))

        # (one accumulator: splitting the chain over two registers measured slower)
        def dots(g):
            if sequential and c == 3 and not ROUNDED_SUM:
                # The last kv block's row sums wait until their B MFMAs are going out (the exponentials of group
                # g are done by then: their packs feed B(3, q) half g >> 1): they fill the gaps of the step's
                # last MFMAs, which have no softmax left to hide, instead of crowding the block's short window.
                for u in range(4):
                    e = 4 * g + u
                    late_sums.append(valu(f"v_add_f32_e32 {L}, {L}, {vr(s + e)}", kL, kL | vset(s + e),
                                          earliest=b_first(c, q, g >> 1)))
                return
            if ROUNDED_SUM:
                for h in range(2):
                    pr = v_p(c, q, g >> 1) + 2 * (g & 1) + h
                    ops.append(valu(f"v_dot2c_f32_bf16_e32 {L}, 0x3f803f80, {vr(pr)}", kL, kL | vset(pr)))
            else:
                for u in range(4):
                    e = 4 * g + u
                    ops.append(valu(f"v_add_f32_e32 {L}, {L}, {vr(s + e)}", kL, kL | vset(s + e)))

        exps(0)
        for g in range(4):
            packs(g)
            if g < 3:
                exps(g + 1)
            dots(g)
        ops[0].earliest = max(ops[0].earliest, a_mfma(c, 7, q) + 4)   # the chain's last result needs 12 wait states
        if c + 2 < 4:
            ops[-1].deadline = min(ops[-1].deadline or (1 << 30), a_mfma(c + 2, 0, q))  # A(c + 2) writes the same S registers
        return ops

    # The softmax chains share their temporaries: one after the other, in the order of the half stages.
    soft = []
    for c in range(4):
        for q in range(2):
            soft.extend(softmax_chain(c, q))
    chains = [soft, [op for _, op in reads]]
    if late_sums:
        chains.append(late_sums)
    # the operand addresses move to the other step buffer behind their last read of the step
    chains.append(address_flips(read_texts, lambda name, at: valu(
        f"v_xor_b32_e32 %[{name}], 0x10000, %[{name}]", {("op", name)}, {("op", name)}, earliest=at)))
    if alibi:
        # chain (1, q): behind the first MFMA of chain (0, q) and before this step's first softmax
        chains.append([Op(lambda e, q=q: bias_ops(e, 1, q, S_CUR[0]), cost=CAP, earliest=2 + q, deadline=a_mfma(1, 0, q) - 6)
                       for q in range(2)])

    # ---- next step's K / V tiles: 16 LDS-direct loads per wave spread over the stream ------------
    vm = []
    k = 0
    for t, gbase in enumerate((S_GK0, S_GK1, S_GV0, S_GV1)):  # half tiles in LDS order
        for i in range(4):
            at = LOAD_FIRST + LOAD_EVERY * k

            # (M0 of load k + 1 is written behind load k; the loop top writes the first one's)
            nxt = None if k == 15 else ((k + 1) // 4) * TILE + ((k + 1) % 4) * 1024

            def emit(e, nxt=nxt, goff="%[g1v]" if i == 1 else f"%[g{i}]", gb=gbase):
                if "vmem" not in DROP:
                    e.lds_direct_load_chained(goff, gb, nxt, S_LDSN)
            vm.append(Op(emit, cost=LOAD_COST, earliest=at, deadline=at + 12))
            k += 1
    chains.append(vm)

    if masked:
        em.valu(f"v_mov_b32_e32 {vr(V_NEGINF)}, 0xff800000", vset(V_NEGINF), set())
    schedule(em, mfmas, chains, CAP_SOFTCAP if softcap else CAP)
    em.drain()
    return em


OUT_OF_LINE = True  # blocks that are skipped unless needed go behind the loop: the common path falls through


def out_of_line(lines):
    """Splits a stream into the common path and the skipped-unless-needed blocks.  Every `branch over the
    block / block / label` group becomes an inverted branch into the block's copy behind the loop, which
    jumps back: the common path then takes no branch and the loop body shrinks to what it executes."""
    inverse = {"s_cbranch_vccz": "s_cbranch_vccnz", "s_cbranch_scc1": "s_cbranch_scc0"}
    hot, cold = [], []
    i = 0
    while i < len(lines):
        parts = lines[i].split()
        if len(parts) == 2 and parts[0] in inverse and ("_late" in parts[1] or "_keep" in parts[1]):
            label = parts[1]
            j = lines.index(label + ":", i)
            there = label.replace(".Lfa_fwd_", ".Lfa_fwd_x")
            hot += [f"{inverse[parts[0]]} {there}", label + ":"]
            cold += [there + ":"] + lines[i + 1:j] + [f"s_branch {label}"]
            i = j + 1
        else:
            hot.append(lines[i])
            i += 1
    return hot, cold


def run_loop(full, masked, alibi=False, softcap=False):
    """One asm statement: a run of consecutive steps [it, it_end) of one work item, all full or a
    single partial one.  At entry the step's K / V tiles are resident in LDS buffer %[buf]."""
    t0, t1, t2, t3 = S_T
    S = SREG
    entry = [f"ds_read_b128 {vr(V_TBL + 4 * i, 4)}, %[tbl] offset:{16 * i}" for i in range(len(TABLE) // 4)]
    entry += ["s_waitcnt lgkmcnt(0)"]  # (the streams count LDS operations from zero)
    entry += [f"v_readfirstlane_b32 {S[n]}, {vr(V_TBL + i)}" for i, n in enumerate(TABLE)]
    entry += [f"v_readfirstlane_b32 {S[n]}, %[{n}]" for n in STATE_IO + STATE_IN]
    entry += [f"v_mov_b32_e32 {vr(V_TAU)}, {TAU}", f"s_mov_b32 {S_PEND[0]}, 0", f"s_mov_b32 {S_PEND[1]}, 0"]
    if alibi:
        pre = Emitter()
        entry += [f"v_readfirstlane_b32 {S_CUR[0]}, %[ka0]", f"v_readfirstlane_b32 {S_CUR[1]}, %[kb0]"]
        for q in range(2):
            bias_ops(pre, 0, q, S_CUR[0])   # (used by the first MFMAs of the loop, more than 20 instructions on)
        entry += pre.out
    elif not softcap:
        entry += [f"v_sub_f32_e32 {vr(V_NEGM + 16 * q + e)}, 0, %[M{q}]" for q in range(2) for e in range(16)]
    top = entry + [".Lfa_fwd_loop_%=:"]
    # on the item's last step the tiles copied "for the next step" are the first step of the next
    # work item (from the table; with no next item they repeat this one's)
    ka, kb_, kglo, kghi, vglo, vghi = S_SEL
    top += [f"s_add_u32 {t0}, {S['it']}, 1", f"s_cmp_eq_u32 {t0}, {S['n_steps']}",
            f"s_cselect_b32 {ka}, {S['kban']}, {S['kba1']}", f"s_cselect_b32 {kb_}, {S['kbbn']}, {S['kbb1']}",
            f"s_cselect_b32 {kglo}, {S['kgn_lo']}, {S['kg_lo']}", f"s_cselect_b32 {kghi}, {S['kgn_hi']}, {S['kg_hi']}",
            f"s_cselect_b32 {vglo}, {S['vgn_lo']}, {S['vg_lo']}", f"s_cselect_b32 {vghi}, {S['vgn_hi']}, {S['vg_hi']}"]
    for pair, (blo, bhi), kb in ((S_GK0, (kglo, kghi), ka), (S_GK1, (kglo, kghi), kb_), (S_GV0, (vglo, vghi), ka),
                                 (S_GV1, (vglo, vghi), kb_)):
        n = int(pair[2:].split(":")[0])
        top += [f"s_lshl_b32 {t2}, {kb}, 14", f"s_lshr_b32 {t3}, {kb}, 18",  # 64 rows x 256 bytes per kv tile
                f"s_add_u32 s{n}, {blo}, {t2}", f"s_addc_u32 s{n + 1}, {bhi}, {t3}"]
    top += [f"s_xor_b32 {t1}, {S['buf']}, 1", f"s_lshl_b32 {t1}, {t1}, 16", f"s_add_u32 {S_LDSN}, {t1}, {S['w4k']}",
            f"s_mov_b32 m0, {S_LDSN}",   # LDS destination of the step's first copy (the streams write the others)
            f"s_cmp_eq_u32 {S['partial']}, 0", "s_cbranch_scc1 .Lfa_fwd_full_%="]
    tail = [
        ".Lfa_fwd_tail_%=:",
        # list entries of the step after the next one, clamped into the list (a second half past its
        # end repeats the last tile: finite data, its keep bits are zero)
        f"s_add_u32 {t0}, {S['it']}, 2",
        f"s_lshl_b32 {t0}, {t0}, 1",
        f"s_sub_u32 {t1}, {S['n_list']}, 1",
        f"s_min_u32 {t2}, {t0}, {t1}",
        f"s_add_u32 {t0}, {t0}, 1",
        f"s_min_u32 {t3}, {t0}, {t1}",
    ] + ([f"s_sub_u32 {t2}, {t1}, {t2}", f"s_sub_u32 {t3}, {t1}, {t3}"] if alibi else []) + [  # (the list is walked from its end)
        f"s_lshl_b32 {t2}, {t2}, 2",
        f"s_lshl_b32 {t3}, {t3}, 2",
        f"v_add_u32_e32 {vr(V_KB2)}, {t2}, %[lst]",
        f"v_add_u32_e32 {vr(V_KB2 + 1)}, {t3}, %[lst]",
        f"ds_read_b32 {vr(V_KB2)}, {vr(V_KB2)}",
        f"ds_read_b32 {vr(V_KB2 + 1)}, {vr(V_KB2 + 1)}",
        "s_waitcnt vmcnt(0) lgkmcnt(0)",
        "s_barrier",
        f"s_add_u32 {S['it']}, {S['it']}, 1",
        f"v_readfirstlane_b32 {S['kba1']}, {vr(V_KB2)}",
        f"v_readfirstlane_b32 {S['kbb1']}, {vr(V_KB2 + 1)}",
        f"s_xor_b32 {S['buf']}, {S['buf']}, 1",
    ]
    if alibi:
        tail += [f"s_mov_b32 {S_CUR[0]}, {ka}", f"s_mov_b32 {S_CUR[1]}, {kb_}"]
    tail += [f"s_cmp_lt_u32 {S['it']}, {S['it_end']}", "s_cbranch_scc1 .Lfa_fwd_loop_%="]
    tail += [f"v_mov_b32_e32 %[{n}], {S[n]}" for n in STATE_IO]
    if OUT_OF_LINE:
        m_hot, m_cold = out_of_line(masked.out)
        f_hot, f_cold = out_of_line(full.out)
        return (top + m_hot + ["s_branch .Lfa_fwd_tail_%=", ".Lfa_fwd_full_%=:"] + f_hot + tail
                + ["s_branch .Lfa_fwd_end_%="] + m_cold + f_cold + [".Lfa_fwd_end_%=:"])
    return top + masked.out + ["s_branch .Lfa_fwd_tail_%=", ".Lfa_fwd_full_%=:"] + full.out + tail


def main():
    global DROP
    here = os.path.dirname(os.path.abspath(__file__))
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("out", nargs="?", default=os.path.join(here, "fwd_tile.inc"))
    ap.add_argument("--drop", default="", help="comma list of mfma,valu,lds,vmem: leave these instruction classes out "
                    "(the stream then computes nothing useful; for timing what bounds it)")
    args = ap.parse_args()
    if args.drop:
        DROP = tuple(x for x in args.drop.split(",") if x)
    with open(args.out, "w") as f:
        f.write("// Generated by gen_fwd_tile.py; do not edit.\n")

        def macro(name, lines):
            f.write(f"#define {name} \\\n")
            f.write(" \\\n".join(f'  "{line}\\n"' for line in lines))
            f.write("\n\n")

        full, masked = build(False), build(True)
        macro("FA_FWD_RUN", run_loop(full, masked))
        macro("FA_FWD_RUN_ALIBI", run_loop(build(False, True), build(True, True), True))
        macro("FA_FWD_RUN_SOFTCAP", run_loop(build(False, softcap=True), build(True, softcap=True), softcap=True))
        for name, em in (("full", full), ("masked", masked)):
            print(f"{args.out}: {name}: {len(em.out)} instructions, {em.stats}", file=sys.stderr)
        macro("FA_FWD_ZERO_ACC", [f"v_accvgpr_write_b32 a{A_O + i}, 0" for i in range(128)])
        # Q^T fragment ks of both q blocks from 8 dword operands (two pinned outputs come first)
        for ks in range(8):
            macro(f"FA_FWD_PUT_{ks}",
                  [f"v_accvgpr_write_b32 a{A_Q + 4 * ks + i}, %{2 + i}" for i in range(4)]
                  + [f"v_accvgpr_write_b32 a{A_Q + 32 + 4 * ks + i}, %{6 + i}" for i in range(4)])
        # accumulator tile t (q block t / 4, d block t % 4) into 16 dword operands (they are read in order:
        # the s_nop of the first one covers the MFMA -> read hazard)
        for t in range(8):
            macro(f"FA_FWD_GET_ACC_{t}", (["s_nop 15"] if t == 0 else []) + [f"v_accvgpr_read_b32 %{i}, a{A_O + 16 * t + i}" for i in range(16)])


if __name__ == "__main__":
    main()
