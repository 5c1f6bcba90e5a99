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
  * the row sum L adds the fp32 values of p.
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
from gfx950_stream import Emitter, ar, aset, vr, vset  # noqa: E402

PREFETCH = 4     # MFMA pairs between the LDS reads of a pair and its MFMAs
LOAD_FIRST = 1   # MFMA slot of the first LDS-direct load of the next step
LOAD_EVERY = 3   # slots between two of them
TAU = "0x40c00000"  # 6.0: M moves when the running maximum relative to it leaves [-6, 6]
DROP = ()        # instruction classes left out (--drop, timing studies only)

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


def v_s(c, x):
    return V_S0 + 32 * (c & 1) + 16 * x


def v_p(c, x, u):
    return V_P0 + 8 * x + 4 * u


def build(masked):
    em = Emitter()
    # MFMA items (2 MFMAs + one staging slot each), in issue order.  The two q blocks of a kv block
    # are processed half a stage apart: E(c, 0) runs under A(c+1)[ks 0-3] and B(c-1, 1), E(c, 1) under
    # A(c+1)[ks 4-7] and B(c, 0), so every softmax has MFMAs of both kinds to hide under.
    pairs = []
    first, last = {}, {}   # MFMA slot range of half stage (c, q)

    def add_A(c, lo, hi):
        for ks in range(lo, hi):
            pairs.append(("A", c, ks))

    def add_B(c, q):
        for u in range(2):
            for j in range(2):
                pairs.append(("B", c, (q, u, j)))

    add_A(0, 0, 8)
    for c in range(4):
        for q in range(2):
            first[(c, q)] = 2 * len(pairs)
            if c < 3:
                add_A(c + 1, 4 * q, 4 * q + 4)
            if q == 1:
                add_B(c, 0)
            elif c > 0:
                add_B(c - 1, 1)
            last[(c, q)] = 2 * len(pairs)
    stage_end = 2 * len(pairs)
    add_B(3, 1)
    n_slots = 2 * len(pairs)
    def half_off(c):
        return (c >> 1) * TILE + (c & 1) * (TILE // 2)

    # Staging registers.  K row fragments rotate through eight 4-register slots.  The V^T fragments of
    # a kv block have fixed places: B(c, 0) loads them, B(c, 1) half a stage later uses them again,
    # and the fragments of block c + 1 are read in once the MFMA of B(c, 1) that used the place has
    # been issued (B(c + 1, 0) follows B(c, 1) at the same distance).
    a_index = {}
    for k, (kind, c, x) in enumerate(pairs):
        if kind == "A":
            a_index[k] = len(a_index)

    def k_slot(k):
        return A_STG + 32 + 4 * (a_index[k] % 8)

    def v_place(u, db):
        return A_STG + 4 * (4 * u + db)

    def pair_loads(k):
        kind, c, x = pairs[k]
        if kind == "A":
            return [(f"ds_read_b128 {ar(k_slot(k), 4)}, %[r{x}] offset:{half_off(c)}", aset(k_slot(k), 4))]
        q, u, j = x
        if q == 1:
            return []
        off = 2 * TILE + half_off(c) + u * 4096
        loads = []
        for db in (2 * j, 2 * j + 1):
            for hi in range(2):
                reg = v_place(u, db) + 2 * hi
                loads.append((f"ds_read_b64_tr_b16 {ar(reg, 2)}, %[t{2 * db + hi}] offset:{off}", aset(reg, 2)))
        return loads

    def pair_mfmas(k):
        kind, c, x = pairs[k]
        out = []
        if kind == "A":
            ks = x
            base = k_slot(k)
            for q in range(2):
                s = v_s(c, q)
                # the chain starts from -M: its result is the score relative to the reference maximum
                cin = V_NEGM + 16 * q if ks == 0 else s
                out.append((vr(s, 16), ar(base, 4), ar(A_Q + 32 * q + 4 * ks, 4), vr(cin, 16), vset(s, 16), aset(base, 4),
                            aset(A_Q + 32 * q + 4 * ks, 4), vset(cin, 16)))
            return out
        q, u, j = x
        p = v_p(c, q, u)
        for db in (2 * j, 2 * j + 1):
            acc = A_O + 64 * q + 16 * db
            vt = v_place(u, db)
            out.append((ar(acc, 16), ar(vt, 4), vr(p, 4), ar(acc, 16), aset(acc, 16), aset(vt, 4), vset(p, 4), aset(acc, 16)))
        return out

    # ---- VALU work of E(c, q): a list of (kind, ...) ------------------------------------------
    T = [V_TMP + i for i in range(10)]
    tag = "m" if masked else "f"

    def softmax_ops(c, q):
        """Online softmax of the lane's 16 scores (relative to M) of q block q in kv block c."""
        s = v_s(c, q)
        M, Mt, L = f"%[M{q}]", f"%[Mt{q}]", f"%[L{q}]"
        kM, kMt, kL = {("op", f"M{q}")}, {("op", f"Mt{q}")}, {("op", f"L{q}")}
        D, AL, negm = V_D + q, V_AL + q, V_NEGM + 16 * q
        ops = []

        def valu(text, dst, src, trans=False):
            ops.append(("valu", text, dst, src, trans))

        def raw(text):
            ops.append(("raw", text))

        if c > 0:
            # M moved while this block's chain was in flight with the old -M: apply the shift now
            raw(f"s_cmp_eq_u32 {S_PEND[q]}, 0")
            raw(f"s_cbranch_scc1 .Lfa_fwd_{tag}_late{c}{q}_%=")
            ops.append(("skip_begin",))
            for e in range(16):
                valu(f"v_sub_f32_e32 {vr(s + e)}, {vr(s + e)}, {vr(D)}", vset(s + e), vset(s + e) | vset(D))
            raw(f"s_mov_b32 {S_PEND[q]}, 0")
            ops.append(("skip_end",))
            ops.append(("label", f".Lfa_fwd_{tag}_late{c}{q}_%=:"))
        if masked:
            for g in range(4):
                for u in range(4):
                    e = 4 * g + u
                    valu(f"v_bfe_i32 {vr(V_MSK + u)}, %[m{2 * q + (c >> 1)}], {16 * (c & 1) + e}, 1", vset(V_MSK + u), set())
                for u in range(4):
                    e = 4 * g + u  # keep ? score : -inf
                    valu(f"v_bfi_b32 {vr(s + e)}, {vr(V_MSK + u)}, {vr(s + e)}, {vr(V_NEGINF)}", vset(s + e),
                         vset(s + e) | vset(V_MSK + u) | vset(V_NEGINF))
        # block maximum of the lane's 16 scores, then across the two half-waves that share the q row
        for i in range(5):
            valu(f"v_max3_f32 {vr(T[i])}, {vr(s + 3 * i)}, {vr(s + 3 * i + 1)}, {vr(s + 3 * i + 2)}", vset(T[i]), vset(s + 3 * i, 3))
        valu(f"v_max3_f32 {vr(T[0])}, {vr(T[0])}, {vr(T[1])}, {vr(T[2])}", vset(T[0]), vset(T[0]) | vset(T[1]) | vset(T[2]))
        valu(f"v_max3_f32 {vr(T[3])}, {vr(T[3])}, {vr(T[4])}, {vr(s + 15)}", vset(T[3]), vset(T[3]) | vset(T[4]) | vset(s + 15))
        valu(f"v_max_f32_e32 {vr(T[0])}, {vr(T[0])}, {vr(T[3])}", vset(T[0]), vset(T[0]) | vset(T[3]))
        valu(f"v_mov_b32_e32 {vr(T[1])}, {vr(T[0])}", vset(T[1]), vset(T[0]))
        raw("s_nop 1")
        valu(f"v_permlane32_swap_b32 {vr(T[0])}, {vr(T[1])}", vset(T[0]) | vset(T[1]), vset(T[0]) | vset(T[1]))
        raw("s_nop 1")
        valu(f"v_max_f32_e32 {vr(T[0])}, {vr(T[0])}, {vr(T[1])}", vset(T[0]), vset(T[0]) | vset(T[1]))
        valu(f"v_max_f32_e32 {Mt}, {Mt}, {vr(T[0])}", kMt, kMt | vset(T[0]))
        # does the running maximum leave [-TAU, TAU] (and is it finite: rows that kept nothing so far stay put)?
        valu(f"v_cmp_gt_f32_e64 vcc, |{Mt}|, {vr(V_TAU)}", set(), kMt | vset(V_TAU))
        if masked:
            valu(f"v_cmp_neq_f32_e64 s[86:87], {Mt}, {vr(V_NEGINF)}", set(), kMt | vset(V_NEGINF))
            raw("s_and_b64 vcc, vcc, s[86:87]")
        raw(f"s_cbranch_vccz .Lfa_fwd_{tag}_keep{c}{q}_%=")
        ops.append(("skip_begin",))
        raw("s_nop 3")
        valu(f"v_cndmask_b32_e32 {vr(D)}, 0, {Mt}, vcc", vset(D), kMt)                 # the lane's shift
        valu(f"v_exp_f32_e64 {vr(AL)}, -{vr(D)}", vset(AL), vset(D), True)
        valu(f"v_sub_f32_e32 {Mt}, {Mt}, {vr(D)}", kMt, kMt | vset(D))
        valu(f"v_add_f32_e32 {M}, {M}, {vr(D)}", kM, kM | vset(D))
        valu(f"v_mul_f32_e32 {L}, {L}, {vr(AL)}", kL, kL | vset(AL))
        for i in range(64):
            t = T[5 + (i % 4)]
            acc = A_O + 64 * q + i
            valu(f"v_accvgpr_read_b32 {vr(t)}, {ar(acc)}", vset(t), aset(acc))
            valu(f"v_mul_f32_e32 {vr(t)}, {vr(t)}, {vr(AL)}", vset(t), vset(t) | vset(AL))
            valu(f"v_accvgpr_write_b32 {ar(acc)}, {vr(t)}", aset(acc), vset(t))
        for e in range(16):
            valu(f"v_sub_f32_e32 {vr(s + e)}, {vr(s + e)}, {vr(D)}", vset(s + e), vset(s + e) | vset(D))
        for e in range(16):
            valu(f"v_sub_f32_e32 {vr(negm + e)}, {vr(negm + e)}, {vr(D)}", vset(negm + e), vset(negm + e) | vset(D))
        if c < 3:
            raw(f"s_mov_b32 {S_PEND[q]}, 1")  # (kv block c + 1 of this step is in flight; block 0 of the next step is not)
        ops.append(("skip_end",))
        ops.append(("label", f".Lfa_fwd_{tag}_keep{c}{q}_%=:"))
        # p = 2^(score - M), packed to bf16 B operands.  The row sum adds the fp32 values in four
        # interleaved partial sums (plain adds hide under the MFMAs; v_dot2c on the packed values
        # measured 9 cycles apiece).
        def exps(g):
            for u in range(4):
                e = 4 * g + u
                valu(f"v_exp_f32_e32 {vr(s + e)}, {vr(s + e)}", vset(s + e), vset(s + e), True)

        def packs(g):
            for h in range(2):
                e = 4 * g + 2 * h
                pr = v_p(c, q, g >> 1) + 2 * (g & 1) + h
                valu(f"v_cvt_pk_bf16_f32 {vr(pr)}, {vr(s + e)}, {vr(s + e + 1)}", vset(pr), vset(s + e, 2))

        def sums(g):
            for u in range(4):
                e = 4 * g + u
                if g == 1:
                    valu(f"v_add_f32_e32 {vr(T[u])}, {vr(s + u)}, {vr(s + e)}", vset(T[u]), vset(s + u) | vset(s + e))
                elif g > 1:
                    valu(f"v_add_f32_e32 {vr(T[u])}, {vr(T[u])}, {vr(s + e)}", vset(T[u]), vset(T[u]) | vset(s + e))

        exps(0)
        for g in range(4):
            if g < 3:
                exps(g + 1)
            sums(g)
            packs(g)
        valu(f"v_add_f32_e32 {vr(T[0])}, {vr(T[0])}, {vr(T[1])}", vset(T[0]), vset(T[0]) | vset(T[1]))
        valu(f"v_add_f32_e32 {vr(T[2])}, {vr(T[2])}, {vr(T[3])}", vset(T[2]), vset(T[2]) | vset(T[3]))
        valu(f"v_add_f32_e32 {vr(T[0])}, {vr(T[0])}, {vr(T[2])}", vset(T[0]), vset(T[0]) | vset(T[2]))
        valu(f"v_add_f32_e32 {L}, {L}, {vr(T[0])}", kL, kL | vset(T[0]))
        return ops

    slot_ops = {m: [] for m in range(n_slots + 1)}
    slot_lds = {m: [] for m in range(n_slots)}
    pre_lds = []
    for c in range(4):
        for q in range(2):
            ops = softmax_ops(c, q)
            lo = first[(c, q)] + 4  # the block's last MFMAs were issued just before: give their results time
            span = last[(c, q)] - lo
            # a branch, the block it may skip and its label stay in one slot (no MFMA or LDS read may
            # end up inside the skipped range); the block counts for nothing when the work is spread
            total = 0
            inside = False
            for op in ops:
                if op[0] == "skip_begin":
                    inside = True
                if not inside and op[0] != "label":
                    total += 1
                if op[0] == "skip_end":
                    inside = False
            done = 0
            pinned = None
            for i, op in enumerate(ops):
                if pinned is None and i + 1 < len(ops) and ops[i + 1][0] == "skip_begin":
                    pinned = lo + (done * span) // total  # (op is the branch)
                slot_ops[pinned if pinned is not None else lo + (done * span) // total].append(op)
                if pinned is None or i + 1 < len(ops) and ops[i + 1][0] == "skip_begin":
                    done += 1
                if op[0] == "label":
                    pinned = None

    for k in range(len(pairs)):
        # (V^T fragments one pair later than K rows: in the last stages, which have no A pairs, the
        # place's previous user is only four pairs ahead and must have been issued)
        at = 2 * (k - (PREFETCH if pairs[k][0] == "A" else PREFETCH - 1))
        if at < 0:
            pre_lds.extend(pair_loads(k))
        else:
            slot_lds[at] = pair_loads(k) + slot_lds[at]

    slot_vmem = {m: [] for m in range(n_slots)}
    k = 0
    for t, gbase in enumerate((S_GK0, S_GK1, S_GV0, S_GV1)):  # half tiles in LDS order
        for i in range(4):
            slot_vmem[LOAD_FIRST + LOAD_EVERY * k].append((t * TILE + i * 1024, "%[g1v]" if i == 1 else f"%[g{i}]", gbase, S_LDSN))
            k += 1

    def emit(op):
        if op[0] == "raw":
            em.raw(op[1])
        elif op[0] == "label":
            em.label(op[1])
        elif op[0] == "skip_begin":
            em.skip_begin()
        elif op[0] == "skip_end":
            em.skip_end()
        elif "valu" not in DROP:
            em.valu(*op[1:])

    if masked:
        em.valu(f"v_mov_b32_e32 {vr(V_NEGINF)}, 0xff800000", vset(V_NEGINF), set())
    for text, dst in pre_lds:
        em.lds_read(text, dst)
    holds = {}  # V^T place -> kv block whose fragment was last read into it
    for k, (kind, c, x) in enumerate(pairs):
        if kind == "B" and x[0] == 0 and 2 * (k - (PREFETCH - 1)) < 0:
            raise AssertionError("V^T fragments are never part of the preamble")
    for m in range(n_slots):
        for ld in slot_vmem[m]:  # (M0 was written in front of the previous MFMA)
            if "vmem" not in DROP:
                em.lds_direct_issue(ld[1], ld[2])
        for text, dst in slot_lds[m]:
            if "lds" not in DROP:
                em.lds_read(text, dst)
        for k, (kind, c, x) in enumerate(pairs):  # bookkeeping of the V^T places (see v_place)
            if kind == "B" and x[0] == 0 and 2 * (k - (PREFETCH - 1)) == m:
                for db in (2 * x[2], 2 * x[2] + 1):
                    holds[(x[1], db)] = c
        kind, c, x = pairs[m // 2]
        if kind == "B":
            db = 2 * x[2] + (m % 2)
            assert holds.get((x[1], db)) == c, f"B({c}, {x[0]}) would multiply with the V^T fragment of block {holds.get((x[1], db))}"
        for ld in slot_vmem.get(m + 1, []):  # (the MFMA below is the wait state between M0 and its load)
            if "vmem" not in DROP:
                em.lds_direct_dest(ld[0], ld[3])
        if "mfma" not in DROP:
            em.mfma(*pair_mfmas(m // 2)[m % 2])
        for op in slot_ops[m]:
            emit(op)
    em.drain()
    return em


def run_loop(full, masked):
    """One asm statement: a run of consecutive steps [it, it_end) of one work item, all full or a
    single partial one.  At entry the step's K / V tiles are resident in LDS buffer %[buf]."""
    t0, t1, t2, t3 = S_T
    S = SREG
    entry = [f"ds_read_b128 {vr(V_TBL + 4 * i, 4)}, %[tbl] offset:{16 * i}" for i in range(len(TABLE) // 4)]
    entry += ["s_waitcnt lgkmcnt(0)"]  # (the streams count LDS operations from zero)
    entry += [f"v_readfirstlane_b32 {S[n]}, {vr(V_TBL + i)}" for i, n in enumerate(TABLE)]
    entry += [f"v_readfirstlane_b32 {S[n]}, %[{n}]" for n in STATE_IO + STATE_IN]
    entry += [f"v_mov_b32_e32 {vr(V_TAU)}, {TAU}", f"s_mov_b32 {S_PEND[0]}, 0", f"s_mov_b32 {S_PEND[1]}, 0"]
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
    tail += [f"v_xor_b32_e32 %[r{i}], 0x10000, %[r{i}]" for i in range(8)]
    tail += [f"v_xor_b32_e32 %[t{i}], 0x10000, %[t{i}]" for i in range(8)]
    tail += [f"s_cmp_lt_u32 {S['it']}, {S['it_end']}", "s_cbranch_scc1 .Lfa_fwd_loop_%="]
    tail += [f"v_mov_b32_e32 %[{n}], {S[n]}" for n in STATE_IO]
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
        for name, em in (("full", full), ("masked", masked)):
            print(f"{args.out}: {name}: {len(em.out)} instructions, {em.stats}", file=sys.stderr)
        macro("FA_FWD_ZERO_ACC", [f"v_accvgpr_write_b32 a{A_O + i}, 0" for i in range(128)])
        # Q^T fragment ks of both q blocks from 8 dword operands (two pinned outputs come first)
        for ks in range(8):
            macro(f"FA_FWD_PUT_{ks}",
                  [f"v_accvgpr_write_b32 a{A_Q + 4 * ks + i}, %{2 + i}" for i in range(4)]
                  + [f"v_accvgpr_write_b32 a{A_Q + 32 + 4 * ks + i}, %{6 + i}" for i in range(4)])
        # accumulator tile t (q block t / 4, d block t % 4) into 16 dword operands
        for t in range(8):
            macro(f"FA_FWD_GET_ACC_{t}", ["s_nop 15"] + [f"v_accvgpr_read_b32 %{i}, a{A_O + 16 * t + i}" for i in range(16)])


if __name__ == "__main__":
    main()
