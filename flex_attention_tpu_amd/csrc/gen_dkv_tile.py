#!/usr/bin/env python3
"""Generator of the hand-scheduled gfx950 instruction stream for one full (unmasked, plain-score)
128 x 128 tile of the bf16 dk/dv kernel.  Writes bwd_dkv_tile.inc: string-literal macros (the stream for
full tiles and the one for partially masked tiles, selected by a scalar branch inside one statement,
plus prologue / epilogue register moves) that bwd_dkv_bf16.hip places inside `asm volatile` statements.

Why generated assembly: with 128 accumulator and 64 K/V operand registers the kernel runs one wave
per SIMD, so MFMA, VALU and LDS work only overlap if they are interleaved inside the wave, and the
register budget only closes with a fixed allocation.  The stream below is a software pipeline over
the tile's four 32-row q blocks c = 0..3:

    A(c): S = Q K^T, dP' = dO V^T - delta  16 MFMAs, operands: 16 ds_read_b128 (rows of Q, dO)
          (LDS holds -lse and -delta; -delta enters through the accumulator input of the dP chain's
          first MFMA)
    E(c): P = exp2(c2 S - lse), dS = P dP'   64 VALU ops; 8 ds_read_b128 (-lse, -delta)
          (c2 = sm_scale log2 e is applied to the fp32 products by the fma that subtracts lse.  Folding it
          into the bf16 K operand instead saves those 16 fmas per block, but rounds every scaled K element
          to bf16 again: the logits then carry an error of about 2e-3 rms with Gaussian tails, which was
          the largest share of the maximum error of dk and dv)
    B(c): dv^T += dO^T P, dk^T += Q^T dS 16 MFMAs, operands: 32 ds_read_b64_tr_b16

    MFMA order:  A0 | A1 | A2 B0 | A3 B1 | B2 | B3      VALU:  - | E0 | E1 | E2 | E3 | -

LDS reads are issued PREFETCH MFMA pairs ahead of their use into a rotating pool of staging
registers; the next step's Q / dO tiles are copied global -> LDS by 16 loads spread over the stream.
The emitter (gfx950_stream.py) inserts the s_nop / s_waitcnt that the hardware hazards require.

Register contract with the C++ side (every asm statement names the accumulation registers with
physical-register constraints; prologue / epilogue macros are generated here too):
    a[0:63]    dv accumulators (4 x 16)      a[64:127]  dk accumulators (4 x 16)
    a[128:159] K fragments (8 x 4)               a[160:191] V fragments (8 x 4)
    %[c2v]     sm_scale log2(e) in every lane (softcap: 2 log2(e) sm_scale / cap)
    v[67:199]  scratch of the run loop and its streams (clobbered), s[60:100], vcc, m0 likewise
    a[192:255] staging slots of the LDS fragments (clobbered): MFMA operands only, so they can be
               AGPRs, and v[192:255] stay with the compiler for what lives across the run loop
    %[r0..r7]  byte address of the lane's row fragment ks in the step's Q half-tile 0
    %[t0..t7]  byte address of the lane's transposed fragment (2 db + hi) in Q half-tile 0
    %[la]      byte address of the lane's first -lse value of the step
    %[partial] flags: bit 0 selects the masked stream, bit 1 says that the run ends its work item and
               that the table's second half (next item's Q, dO, row bases, first q block) is valid
    %[g0..g3]  the lane's byte offsets inside a global half tile for the wave's four 1 KB blocks;
    %[gq0], %[gq1], %[gd0], %[gd1]  global addresses (SGPR pairs) of the next step's Q / dO half tiles;
    %[ldsn]    LDS byte address of the wave's first block in the next step's buffer
    %[m0], %[m1]  (masked stream only) the lane's keep bits: bit 16 (c & 1) + e of m[c >> 1] is
               element e of the S accumulator of q block c; dropped elements get P = 0
LDS layout of one step buffer (bytes): Q half 0, Q half 1, dO half 0, dO half 1 (16 KiB each);
-lse [128] floats, -delta 1 KiB after it.
"""
import argparse
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from gfx950_stream import Emitter, Op, ar, aset, address_flips, schedule, vr, vset  # noqa: E402

NSLOT = 8        # staging slots of 8 registers
MIN_AHEAD = 2    # MFMA pairs at least between the LDS reads of a pair and its MFMAs
WAIT_OLD = 20    # a wait for LDS data also covers younger reads issued at least this many instructions ago
CAP = 6          # instructions the scheduler puts between two MFMAs unless deadlines force more
LOAD_FIRST = 0   # MFMA gap from which the first LDS-direct load of the next step may go out
LOAD_EVERY = 3   # gaps between two of them
LOAD_COST = 3    # share of an MFMA gap one of them takes
LDS_COST = 1     # share of an MFMA gap an LDS read takes
TRANS_COST = 2   # share of an MFMA gap a transcendental takes (it holds the wave's issue for two slots)
DROP = ()        # instruction classes left out (--drop, timing studies only)
DS_COST = 3      # share of an MFMA gap a dS store takes

TILE = 16384
# Scalar registers owned by the run loop (all clobbered).  The compiler hands scalars to an asm
# statement unreliably once many are live (it may keep a uniform value in a VGPR and print that
# VGPR for an "s" operand), so the statement takes none: work-group constants come from a 16-dword
# per-wave table in LDS, the loop state from VGPR operands, both through v_readfirstlane_b32.
TABLE = ["n_tiles", "gmax", "sq", "w4k", "na2", "lsew", "idx_lo", "idx_hi", "qg_lo", "qg_hi", "dog_lo", "dog_hi",
         "rowa_lo", "rowa_hi", "rowb_lo", "rowb_hi"]  # order of the table's dwords
SREG = {"n_tiles": "s60", "gmax": "s61", "sq": "s62", "w4k": "s63", "na2": "s64", "lsew": "s65",
        "idx_lo": "s66", "idx_hi": "s67", "qg_lo": "s68", "qg_hi": "s69", "dog_lo": "s70", "dog_hi": "s71",
        "rowa_lo": "s72", "rowa_hi": "s73", "rowb_lo": "s74", "rowb_hi": "s75",
        "it": "s76", "p1": "s77", "g1": "s78", "p2": "s79", "qb1": "s80", "buf": "s81", "it_end": "s82", "partial": "s83",
        "idx": "s[66:67]"}
STATE_IO = ["it", "p1", "g1", "p2", "qb1", "buf"]   # VGPR operands read at entry, written back at exit
STATE_IN = ["it_end", "partial"]                    # VGPR operands read at entry
V_TBL = 72      # 16 scratch VGPRs the table is read into at entry
S_T = ["s84", "s85", "s86", "s87"]
S_GQ0, S_GQ1, S_GD0, S_GD1, S_RA, S_RB = "s[88:89]", "s[90:91]", "s[92:93]", "s[94:95]", "s[96:97]", "s[98:99]"
S_LDSN = "s100"
S_KC = "s101"     # (position-bias variant) 128 kb + 64: the middle of the item's kv tile
# Softcap variant, s' = cap tanh(s / cap): the chain's result times 2 log2(e) sm_scale / cap (%[c2v]) is u with
# e^(2 s / cap) = 2^u; r = 1 / (2^u + 1) gives tanh = 1 - 2 r and the exponent
# cap' - lse - 2 cap' r with cap' = cap log2(e) (LDS holds cap' - lse; s64 = cap', s101 = -2 cap'), and
# ds'/ds = 1 - tanh^2 = 4 r (1 - r), whose factor 4 the epilogue applies to dk.
S_CAP, S_K2 = "s64", "s101"
CAP_SOFTCAP = 8   # instructions per MFMA gap in the softcap variant (8 VALU ops per element instead of 2)
# dS export variant: the step's bf16 dS (the B operand registers of the dk product) also goes to a buffer in
# global memory, one 32 KB block per (query head, kept tile pair), from which the dq pass takes it.  The blocks of
# a head are ordered kv tile by kv tile and along each kv tile's q list.  Block of the step: item base + ((head
# inside the group) pairs + (place in the q list)) 32 KB; wave w writes bytes [8192 w, + 8192),
# 1 KB per (q block c, half u) at (2 c + u) 1024, lane L at 16 (2 (L % 32) + L / 32).
S_DSB, S_PAIRS, S_DS, S_DSN = "s[52:53]", "s54", "s[56:57]", "s[58:59]"
V_QB2 = 67      # q block index of the step after the next one, across the stream
ROW_SLOT = 28   # MFMA slot at which the next step's lse / delta values are turned around
V_ROW = 144     # 4 temporaries for that, inside pb[1] (first written by E(1), after ROW_SLOT)
V_S = [72, 104]
V_DP = [88, 120]
V_PB = 136
V_DSB = 152
V_LSE = 168   # -lse of the 16 q rows of a block: accumulator input of the first MFMA of its S chain
V_DL = 184    # -delta of the 16 q rows of a block, for the dP chain likewise
A_STG = 192   # 8 staging slots x 8 registers for LDS fragments: AGPRs, which leaves v[192:255] to the compiler
V_TMP = 68    # 4 temporaries of the masked variant
DL_OFFSET = 1024


def build(masked, alibi=False, softcap=False, export=False):
    em = Emitter()
    em.wait_old = WAIT_OLD

    # ---- MFMA pairs in issue order -------------------------------------------------------
    pairs = []
    def add_A(c):
        for ks in range(8):
            pairs.append(("A", c, ks))
    def add_B(c):
        for u in range(2):
            for db in range(4):
                pairs.append(("B", c, (u, db)))
    add_A(0); add_A(1); add_A(2); add_B(0); add_A(3); add_B(1); add_B(2); add_B(3)
    n_mfma = 2 * len(pairs)
    idx = {}  # (kind, c, x) -> number of the pair's first MFMA
    for k, key in enumerate(pairs):
        idx[key] = 2 * k
    first_A = {c: idx[("A", c, 0)] for c in range(4)}
    last_A = {c: idx[("A", c, 7)] + 1 for c in range(4)}
    first_B = {(c, u): idx[("B", c, (u, 0))] for c in range(4) for u in range(2)}
    last_B = {(c, u): idx[("B", c, (u, 3))] + 1 for c in range(4) for u in range(2)}

    def half_off(c):
        return (c >> 1) * TILE + (c & 1) * (TILE // 2)

    def pair_loads(k):
        kind, c, x = pairs[k]
        base = A_STG + 8 * (k % NSLOT)
        loads = []
        if kind == "A":
            ks = x
            loads.append((f"ds_read_b128 {ar(base, 4)}, %[r{ks}] offset:{half_off(c)}", aset(base, 4)))
            loads.append((f"ds_read_b128 {ar(base + 4, 4)}, %[r{ks}] offset:{2 * TILE + half_off(c)}", aset(base + 4, 4)))
        else:
            u, db = x
            off = half_off(c) + u * 4096
            for which, reg0 in ((2 * TILE, base), (0, base + 4)):  # dO fragment, then Q fragment
                for hi in range(2):
                    loads.append((f"ds_read_b64_tr_b16 {ar(reg0 + 2 * hi, 2)}, %[t{2 * db + hi}] offset:{which + off}",
                                  aset(reg0 + 2 * hi, 2)))
        return loads

    def pair_mfmas(k):
        kind, c, x = pairs[k]
        base = A_STG + 8 * (k % NSLOT)
        if kind == "A":
            ks = x
            s, dp = V_S[c & 1], V_DP[c & 1]
            cin = s
            cdn = V_DL if ks == 0 else dp
            first = ((vr(s, 16), ar(base, 4), ar(128 + 4 * ks, 4), "0", vset(s, 16), aset(base, 4), aset(128 + 4 * ks, 4), set())
                     if ks == 0 else
                     (vr(s, 16), ar(base, 4), ar(128 + 4 * ks, 4), vr(cin, 16), vset(s, 16), aset(base, 4), aset(128 + 4 * ks, 4),
                      vset(cin, 16)))
            return [
                first,
                (vr(dp, 16), ar(base + 4, 4), ar(160 + 4 * ks, 4), vr(cdn, 16), vset(dp, 16), aset(base + 4, 4),
                 aset(160 + 4 * ks, 4), vset(cdn, 16)),
            ]
        u, db = x
        pb = V_PB + 8 * (c & 1) + 4 * u
        dsb = V_DSB + 8 * (c & 1) + 4 * u
        return [
            (ar(16 * db, 16), ar(base, 4), vr(pb, 4), ar(16 * db, 16), aset(16 * db, 16), aset(base, 4), vset(pb, 4),
             aset(16 * db, 16)),
            (ar(64 + 16 * db, 16), ar(base + 4, 4), vr(dsb, 4), ar(64 + 16 * db, 16), aset(64 + 16 * db, 16),
             aset(base + 4, 4), vset(dsb, 4), aset(64 + 16 * db, 16)),
        ]

    mfmas = [pair_mfmas(k)[j] for k in range(len(pairs)) for j in range(2)]
    if "mfma" in DROP:
        mfmas = []
        n_gaps = n_mfma

    def valu(text, dst, src, trans=False, **kw):
        return Op((lambda e: e.valu(text, dst, src, trans)) if "valu" not in DROP else (lambda e: None),
                  cost=TRANS_COST if trans else 1, **kw)

    def lds(text, dst, **kw):
        return Op((lambda e: e.lds_read(text, dst)) if "lds" not in DROP else (lambda e: None), cost=LDS_COST, **kw)

    chains = []
    e_chains = []
    state = {"direct": 0, "stores_behind": 0}

    def ds_store(c, u, reg):
        # One 16-byte store per lane and 16-row half, once the half's second group is converted.  (Measured: a store
        # costs the wave about 46 cycles of issue whatever its cache policy bits; two 8-byte stores per half cost more.)
        def emit(e):
            if "vmem" in DROP:
                return
            e.vmem_store(f"global_store_dwordx4 %[dsv], {vr(reg, 4)}, {S_DS} offset:{(2 * c + u) * 1024 - 4096}", vset(reg, 4))
            state["direct"] += 1
            state["stores_behind"] += 1
        return Op(emit, cost=DS_COST, deadline=n_mfma)

    def lse_read(c, g):
        return lds(f"ds_read_b128 {vr(V_LSE + 4 * g, 4)}, %[la] offset:{(32 * c + 8 * g) * 4}", vset(V_LSE + 4 * g, 4))

    # ---- E(c): element-wise work between the block's S / dP chains and its B products -------
    for c in range(4):
        s, dp = V_S[c & 1], V_DP[c & 1]
        ops = []
        for g in range(4):
            c2v = {("op", "c2v")}
            for u in range(4):
                e = 4 * g + u
                if softcap:
                    ops.append(valu(f"v_mul_f32_e32 {vr(s + e)}, %[c2v], {vr(s + e)}", vset(s + e), vset(s + e) | c2v))
                else:
                    ops.append(valu(f"v_fma_f32 {vr(s + e)}, {vr(s + e)}, %[c2v], {vr(V_LSE + e)}", vset(s + e),
                                    vset(s + e) | vset(V_LSE + e) | c2v))
            if not softcap and c < 3:
                ops.append(lse_read(c + 1, g))   # (the next block's row values take the registers just used)
            for u in range(4):
                e = 4 * g + u
                ops.append(valu(f"v_exp_f32_e32 {vr(s + e)}, {vr(s + e)}", vset(s + e), vset(s + e), True))
            if softcap:
                # 2^u -> r = 1 / (2^u + 1); dP' r (1 - r); exponent (cap' - lse) - 2 cap' r -> P
                for text, trans in (("v_add_f32_e32 {s}, 1.0, {s}", False), ("v_rcp_f32_e32 {s}, {s}", True)):
                    for u in range(4):
                        e = 4 * g + u
                        ops.append(valu(text.format(s=vr(s + e)), vset(s + e), vset(s + e), trans))
                for u in range(4):
                    e = 4 * g + u
                    ops.append(valu(f"v_mul_f32_e32 {vr(dp + e)}, {vr(dp + e)}, {vr(s + e)}", vset(dp + e), vset(dp + e) | vset(s + e)))
                for u in range(4):
                    e = 4 * g + u
                    ops.append(valu(f"v_fma_f32 {vr(dp + e)}, -{vr(dp + e)}, {vr(s + e)}, {vr(dp + e)}", vset(dp + e), vset(dp + e) | vset(s + e)))
                for u in range(4):
                    e = 4 * g + u
                    ops.append(valu(f"v_fma_f32 {vr(s + e)}, {vr(s + e)}, {S_K2}, {vr(V_LSE + e)}", vset(s + e), vset(s + e) | vset(V_LSE + e)))
                if c < 3:
                    ops.append(lse_read(c + 1, g))   # (the next block's row values take the registers just used)
                for u in range(4):
                    e = 4 * g + u
                    ops.append(valu(f"v_exp_f32_e32 {vr(s + e)}, {vr(s + e)}", vset(s + e), vset(s + e), True))
            if masked:
                # keep bit of element e of block c: bit 16 (c & 1) + e of %[m0] (c < 2) or %[m1]
                for u in range(4):
                    e = 4 * g + u
                    tmp = V_TMP + u
                    ops.append(valu(f"v_bfe_i32 {vr(tmp)}, %[m{c >> 1}], {16 * (c & 1) + e}, 1", vset(tmp), set()))
                for u in range(4):
                    e = 4 * g + u
                    tmp = V_TMP + u
                    ops.append(valu(f"v_and_b32_e32 {vr(s + e)}, {vr(s + e)}, {vr(tmp)}", vset(s + e), vset(s + e) | vset(tmp)))
            for u in range(4):
                e = 4 * g + u
                ops.append(valu(f"v_mul_f32_e32 {vr(dp + e)}, {vr(s + e)}, {vr(dp + e)}", vset(dp + e), vset(dp + e) | vset(s + e)))
            # bf16x8 operand u2 = g >> 1, registers 2 (g & 1) + {0, 1} hold elements (0,1), (2,3) of the group.
            # The registers are those of block c - 2: its B MFMAs that read them must have been issued;
            # and this block's B MFMAs of half u2 wait for them.
            u2 = g >> 1
            pb = V_PB + 8 * (c & 1) + 4 * u2 + 2 * (g & 1)
            dsb = V_DSB + 8 * (c & 1) + 4 * u2 + 2 * (g & 1)
            war = last_B[(c - 2, u2)] + 1 if c >= 2 else 0
            for h in range(2):
                e = 4 * g + 2 * h
                ops.append(valu(f"v_cvt_pk_bf16_f32 {vr(pb + h)}, {vr(s + e)}, {vr(s + e + 1)}", vset(pb + h), vset(s + e, 2),
                                earliest=war, deadline=first_B[(c, u2)] - 1))
                ops.append(valu(f"v_cvt_pk_bf16_f32 {vr(dsb + h)}, {vr(dp + e)}, {vr(dp + e + 1)}", vset(dsb + h), vset(dp + e, 2),
                                earliest=war, deadline=first_B[(c, u2)] - 1))
            if export and (g & 1):
                ops.append(ds_store(c, u2, V_DSB + 8 * (c & 1) + 4 * u2))
        ops[0].earliest = last_A[c] + 4            # the chains' last results need 12 wait states
        if c + 2 < 4:
            last_cvt = ops[-2] if export else ops[-1]
            last_cvt.deadline = min(last_cvt.deadline, first_A[c + 2])  # A(c + 2) writes the same S / dP registers
        e_chains.append(ops)
    # one chain: block c + 1 must not read its row values before block c has put them there
    chains.append([op for ops in e_chains for op in ops])

    # ---- LDS reads -----------------------------------------------------------------------------
    # operand fragments of the MFMA pairs, in the order of their use: not before the pair that had
    # the staging slot has been issued, at least MIN_AHEAD pairs before their own
    reads = []
    read_texts = []
    for k in range(len(pairs)):
        for text, dst in pair_loads(k):
            reads.append(lds(text, dst, earliest=max(0, 2 * (k - NSLOT) + 2), deadline=max(0, 2 * (k - MIN_AHEAD))))
            read_texts.append((text, max(0, 2 * (k - MIN_AHEAD))))
    chains.append(reads)
    # the operand addresses move to the other step buffer behind their last read of the step
    chains.append(address_flips(read_texts, lambda name, at: valu(
        f"v_xor_b32_e32 %[{name}], 0x10000, %[{name}]", {("op", name)}, {("op", name)}, earliest=at)))
    # -lse and -delta of block c: behind the first MFMAs of A(c - 1), which read the registers, and
    # well before the first MFMAs of A(c)
    rows = []
    for c in range(4):
        for g in range(4):
            for reg, off in ((V_LSE, 0), (V_DL, DL_OFFSET)):
                if reg == V_LSE:
                    continue   # (used by E(c), not by the chain: read there, block 0 below)
                rows.append(lds(f"ds_read_b128 {vr(reg + 4 * g, 4)}, %[la] offset:{(32 * c + 8 * g) * 4 + off}", vset(reg + 4 * g, 4),
                                earliest=first_A[c - 1] + 6 if c else 0, deadline=max(0, first_A[c] - 6)))
    chains.append(rows)
    first_rows = [lse_read(0, g) for g in range(4)]
    first_rows[-1].deadline = last_A[0]
    chains.append(first_rows)

    # ---- next step's Q / dO tiles: 16 LDS-direct loads per wave spread over the stream ----------
    # (issued back to back they hold the wave for about a thousand cycles: one CU moves 64 B / clk)
    # (vector-memory operations complete in issue order: one count of those issued so far, and the text index of
    # the last LDS-direct load, behind which only dS stores are open at the end of the stream)

    # (M0 of load k + 1 is written behind load k; the loop top writes the first one's)
    def direct(k, goff, gbase):
        nxt = None if k == 15 else ((k + 1) // 4) * TILE + ((k + 1) % 4) * 1024

        def emit(e):
            if "vmem" in DROP:
                return
            e.lds_direct_load_chained(goff, gbase, nxt, S_LDSN)
            state["direct"] += 1
            state["stores_behind"] = 0
        return emit

    vm = []
    k = 0
    for t, gbase in enumerate((S_GQ0, S_GQ1, S_GD0, S_GD1)):  # half tiles in LDS order
        for i in range(4):
            at = LOAD_FIRST + LOAD_EVERY * k
            vm.append(Op(direct(k, "%[g1v]" if i == 1 else f"%[g{i}]", gbase), cost=LOAD_COST, earliest=at, deadline=at + 12))
            k += 1
    chains.append(vm)

    def row_turnaround(e):
        if "vmem" in DROP:
            return
        # The two per-row values this lane fetched at the top of the step (older than every
        # LDS-direct load) have arrived once at most as many vector-memory operations are open as
        # LDS-direct loads were issued.  Waves 0, 1: (l, m) -> -lse = -m log2(e) - log2(l), -inf where
        # l = 0; waves 2, 3: -delta (%[lsew] is non-zero resp. zero).  One LDS store into the next buffer.
        ra_, rb_, rt_, inf_ = V_ROW, V_ROW + 1, V_ROW + 2, V_ROW + 3
        e.raw(f"s_waitcnt vmcnt({state['direct']})")
        # (-lse by one fused multiply-add, m (-log2 e) - log2 l: the same rounding as the kernel's own set-up of an
        # item's first step, so that a step's row values do not depend on who prepared them)
        e.valu(f"v_log_f32_e32 {vr(rt_)}, {vr(ra_)}", vset(rt_), vset(ra_), True)
        e.raw(f"s_mov_b32 {S_T[1]}, 0xbfb8aa3b")
        e.valu(f"v_mov_b32_e32 {vr(inf_)}, 0xff800000", vset(inf_), set())
        e.valu(f"v_fma_f32 {vr(rt_)}, {vr(rb_)}, {S_T[1]}, -{vr(rt_)}", vset(rt_), vset(rt_) | vset(rb_))
        e.valu(f"v_cmp_lt_f32_e32 vcc, 0, {vr(ra_)}", set(), vset(ra_))
        e.valu(f"v_cndmask_b32_e32 {vr(rt_)}, {vr(inf_)}, {vr(rt_)}, vcc", vset(rt_), vset(rt_) | vset(inf_))
        if softcap:
            e.valu(f"v_add_f32_e32 {vr(rt_)}, {S_CAP}, {vr(rt_)}", vset(rt_), vset(rt_))   # cap' - lse
        if alibi:
            # + slope log2(e) (j0 - i) for query row i = 128 qb1 + row of the next step, relative to the
            # middle j0 of the kv tile (s64 holds -slope log2 e): the key's share 2^(slope log2(e) (j - j0))
            # is a factor of whole dk / dv rows, which the epilogue applies
            e.raw(f"s_lshl_b32 {S_T[0]}, s80, 7")
            e.raw(f"s_sub_i32 {S_T[0]}, {S_T[0]}, {S_KC}")
            e.valu(f"v_lshrrev_b32_e32 {vr(inf_)}, 2, %[tid4]", vset(inf_), set())
            e.valu(f"v_add_u32_e32 {vr(inf_)}, {S_T[0]}, {vr(inf_)}", vset(inf_), vset(inf_))
            e.valu(f"v_cvt_f32_i32_e32 {vr(inf_)}, {vr(inf_)}", vset(inf_), vset(inf_))
            e.valu(f"v_fma_f32 {vr(rt_)}, {vr(inf_)}, s64, {vr(rt_)}", vset(rt_), vset(rt_) | vset(inf_))
        e.raw("s_cmp_lg_u32 s65, 0")
        e.raw("s_cselect_b64 vcc, -1, 0")
        e.raw("s_nop 3")
        e.valu(f"v_xor_b32_e32 {vr(ra_)}, 0x80000000, {vr(ra_)}", vset(ra_), vset(ra_))
        e.valu(f"v_cndmask_b32_e32 {vr(rt_)}, {vr(ra_)}, {vr(rt_)}, vcc", vset(rt_), vset(rt_) | vset(ra_))
        e.lds_write(f"ds_write_b32 %[lw], {vr(rt_)}", vset(rt_))

    # V_ROW lies inside pb[1] (first written by E(1)): the turn-around runs before E(1) may start
    chains.append([Op(row_turnaround, cost=8, earliest=ROW_SLOT, deadline=last_A[1] + 3)])

    schedule(em, mfmas, chains, CAP_SOFTCAP if softcap else CAP)
    em.drain()
    if export:
        # the step's copies have landed once only the stores issued behind the last of them are open
        em.raw(f"s_waitcnt vmcnt({state['stores_behind']})")
    return em


def run_loop(full, masked, alibi=False, softcap=False, export=False):
    """One asm statement: a run of consecutive steps [it, it_end) of one work-group, all full or a
    single partial one.  At entry the step's Q / dO tiles and row values are resident in LDS buffer
    s81; each pass computes the next step's addresses, streams the tile (which copies the next
    step's data into the other buffer), synchronises the work-group and advances."""
    t0, t1, t2, t3 = S_T
    lo = lambda pair: pair[2:].split(":")[0]  # "s[88:89]" -> "88"
    entry = [f"ds_read_b128 {vr(V_TBL + 4 * i, 4)}, %[tbl] offset:{16 * i}" for i in range(4)]
    entry += ["s_waitcnt lgkmcnt(0)"]  # (the streams count LDS operations from zero)
    entry += [f"v_readfirstlane_b32 {SREG[n]}, {vr(V_TBL + i)}" for i, n in enumerate(TABLE)]
    entry += [f"v_readfirstlane_b32 {SREG[n]}, %[{n}]" for n in STATE_IO + STATE_IN]
    if alibi:
        entry += [f"v_readfirstlane_b32 {S_KC}, %[kc]"]
    if softcap:
        entry += [f"v_readfirstlane_b32 {S_K2}, %[k2]"]
    assert not (alibi and export)
    switch = ([f"ds_read_b64 {vr(V_TBL + 10, 2)}, %[tbl] offset:104"] if alibi or export else [])
    switch_sgprs = ([f"v_readfirstlane_b32 s64, {vr(V_TBL + 10)}", f"v_readfirstlane_b32 {S_KC}, {vr(V_TBL + 11)}"] if alibi else [])
    ds_next = []
    if export:
        # table dwords 28-30: the item's first dS block (two dwords: first query head of the group, first entry of the
        # kv tile's q list), blocks per head (the kept tile pairs of the map); dwords 26, 27: the next item's first dS
        # block; %[dslo], %[dshi]: the block of the run's first step
        entry = ([f"ds_read_b128 {vr(V_TBL + 16, 4)}, %[tbl] offset:112"] + entry
                 + [f"v_readfirstlane_b32 s{52 + i}, {vr(V_TBL + 16 + i)}" for i in range(4)]
                 + ["v_readfirstlane_b32 s56, %[dslo]", "v_readfirstlane_b32 s57, %[dshi]"])
        switch_sgprs = [f"v_readfirstlane_b32 s52, {vr(V_TBL + 10)}", f"v_readfirstlane_b32 s53, {vr(V_TBL + 11)}"]
        # dS block of the next step: item base + (min(g1, gmax) pairs + p1) 32 KB: the blocks of a kv tile follow its
        # q list (p1 = the next step's place in it; 0 where the next step is the next item's first)
        ds_next = [f"s_min_u32 {t0}, s78, s61", f"s_mul_i32 {t0}, {t0}, {S_PAIRS}",
                   f"s_add_u32 {t0}, {t0}, s77", f"s_lshl_b32 {t2}, {t0}, 15", f"s_lshr_b32 {t3}, {t0}, 17",
                   f"s_add_u32 s58, s52, {t2}", f"s_addc_u32 s59, s53, {t3}"]
    top = entry + [
        ".Lfa_dkv_loop_%=:",
        # The last step of the run that ends an item (bit 1 of the flags) copies the next item's first
        # step: that item's bases (second half of the table) and first q block replace this item's.
        f"s_add_u32 {t0}, s76, 1",
        f"s_cmp_lg_u32 {t0}, s82",
        "s_cbranch_scc1 .Lfa_dkv_same_%=",
        "s_bitcmp0_b32 s83, 1",
        "s_cbranch_scc1 .Lfa_dkv_same_%=",
        f"ds_read_b128 {vr(V_TBL, 4)}, %[tbl] offset:64",
        f"ds_read_b128 {vr(V_TBL + 4, 4)}, %[tbl] offset:80",
        f"ds_read_b32 {vr(V_TBL + 8)}, %[tbl] offset:96",
    ] + switch + [
        "s_waitcnt lgkmcnt(0)",
    ] + [f"v_readfirstlane_b32 s{68 + i}, {vr(V_TBL + i)}" for i in range(8)] + switch_sgprs + [
        f"v_readfirstlane_b32 s80, {vr(V_TBL + 8)}",
        "s_mov_b32 s78, 0",
        ".Lfa_dkv_same_%=:",
    ] + ds_next + [
        # row of the next step relative to the first head of the group: min(g1, gmax) Sq + 128 qb1
        f"s_min_u32 {t0}, s78, s61",
        f"s_mul_i32 {t0}, {t0}, s62",
        f"s_lshl_b32 {t1}, s80, 7",
        f"s_add_u32 {t0}, {t0}, {t1}",
        f"s_lshl_b32 {t2}, {t0}, 8",
        f"s_lshr_b32 {t3}, {t0}, 24",
    ]
    for pair, base in ((S_GQ0, "qg"), (S_GD0, "dog")):
        n = int(lo(pair))
        top += [f"s_add_u32 s{n}, {SREG[base + '_lo']}, {t2}", f"s_addc_u32 s{n + 1}, {SREG[base + '_hi']}, {t3}",
                f"s_add_u32 s{n + 2}, s{n}, 0x4000", f"s_addc_u32 s{n + 3}, s{n + 1}, 0"]
    top += [f"s_lshl_b32 {t2}, {t0}, 2", f"s_lshr_b32 {t3}, {t0}, 30"]
    for pair, base in ((S_RA, "rowa"), (S_RB, "rowb")):
        n = int(lo(pair))
        top += [f"s_add_u32 s{n}, {SREG[base + '_lo']}, {t2}", f"s_addc_u32 s{n + 1}, {SREG[base + '_hi']}, {t3}"]
    top += [
        f"s_xor_b32 {t1}, s81, 1",
        f"s_lshl_b32 {t1}, {t1}, 16",
        f"s_add_u32 {S_LDSN}, {t1}, s63",
        f"s_mov_b32 m0, {S_LDSN}",   # LDS destination of the step's first copy (the streams write the others)
        # q block of the step after the next one (the list position wraps inside the list: always valid)
        # (a vector load: an open scalar load would disturb the streams' lgkmcnt bookkeeping)
        f"s_lshl_b32 {t1}, s79, 2",
        f"v_mov_b32_e32 {vr(V_QB2)}, {t1}",
        f"global_load_dword {vr(V_QB2)}, {vr(V_QB2)}, s[66:67]",
        f"global_load_dword {vr(V_ROW)}, %[tid4], {S_RA}",
        f"global_load_dword {vr(V_ROW + 1)}, %[tid4], {S_RB}",
        "s_bitcmp0_b32 s83, 0",
        "s_cbranch_scc1 .Lfa_dkv_full_%=",
    ]
    tail = [
        ".Lfa_dkv_tail_%=:",
        # (dS stores issued behind the step's last copy may stay open: the streams wait for the copies themselves)
        "s_waitcnt lgkmcnt(0)" if export else "s_waitcnt vmcnt(0) lgkmcnt(0)",
        "s_barrier",
    ] + (["s_mov_b64 s[56:57], s[58:59]"] if export else []) + [
        "s_add_u32 s76, s76, 1",
        f"v_readfirstlane_b32 s80, {vr(V_QB2)}",
        "s_add_u32 s77, s77, 1",
        "s_cmp_eq_u32 s77, s60",
        "s_cselect_b32 s77, 0, s77",
        f"s_cselect_b32 {t0}, 1, 0",
        f"s_add_u32 s78, s78, {t0}",
        "s_add_u32 s79, s79, 1",
        "s_cmp_eq_u32 s79, s60",
        "s_cselect_b32 s79, 0, s79",
        "s_xor_b32 s81, s81, 1",
    ]
    tail += ["v_xor_b32_e32 %[la], 0x200, %[la]", "v_xor_b32_e32 %[lw], 0x200, %[lw]",
             "s_cmp_lt_u32 s76, s82", "s_cbranch_scc1 .Lfa_dkv_loop_%="]
    tail += [f"v_mov_b32_e32 %[{n}], {SREG[n]}" for n in STATE_IO]
    return (top + masked.out + ["s_branch .Lfa_dkv_tail_%=", ".Lfa_dkv_full_%=:"] + full.out + tail)


def main():
    global DROP
    here = os.path.dirname(os.path.abspath(__file__))
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("out", nargs="?", default=os.path.join(here, "bwd_dkv_tile.inc"))
    ap.add_argument("--drop", default="", help="comma list of mfma,valu,lds,vmem: leave these instruction classes out "
                    "(the stream then computes nothing useful; for timing what bounds it)")
    args = ap.parse_args()
    if args.drop:
        DROP = tuple(x for x in args.drop.split(",") if x)
    path = args.out
    with open(path, "w") as f:
        f.write("// Generated by gen_dkv_tile.py; do not edit.\n")
        # one statement for both kinds of tile: a second asm statement on another control-flow
        # path makes the compiler shuffle the pinned registers around each of them
        full, masked = build(False), build(True)
        for name, alibi, softcap, export in (("FA_DKV_RUN", False, False, False), ("FA_DKV_RUN_ALIBI", True, False, False),
                                             ("FA_DKV_RUN_SOFTCAP", False, True, False), ("FA_DKV_RUN_DS", False, False, True),
                                             ("FA_DKV_RUN_SOFTCAP_DS", False, True, True)):
            lines = run_loop(build(False, alibi, softcap, export), build(True, alibi, softcap, export), alibi, softcap, export)
            f.write(f"#define {name} \\\n")
            f.write(" \\\n".join(f'  "{line}\\n"' for line in lines))
            f.write("\n\n")
        for name, em in (("full", full), ("masked", masked)):
            print(f"{path}: {name}: {len(em.out)} instructions, {em.stats}", file=sys.stderr)

        def macro(name, lines):
            f.write(f"#define {name} \\\n")
            f.write(" \\\n".join(f'  "{line}\\n"' for line in lines))
            f.write("\n\n")

        # accumulators to zero (prologue)
        macro("FA_DKV_ZERO_ACC", [f"v_accvgpr_write_b32 a{i}, 0" for i in range(128)])
        # K / V fragment ks from 8 dword operands (prologue)
        for ks in range(8):
            macro(f"FA_DKV_PUT_KV_{ks}",
                  [f"v_accvgpr_write_b32 a{128 + 4 * ks + i}, %{2 + i}" for i in range(4)]
                  + [f"v_accvgpr_write_b32 a{160 + 4 * ks + i}, %{6 + i}" for i in range(4)])
        # accumulator tile t (0-3 dv, 4-7 dk) into 16 dword operands (epilogue); the s_nop of the
        # first one covers the MFMA -> read hazard of the last tile stream
        for t in range(8):
            macro(f"FA_DKV_GET_ACC_{t}", (["s_nop 15"] if t == 0 else []) + [f"v_accvgpr_read_b32 %{i}, a{16 * t + i}" for i in range(16)])
        # (operand numbers: PUT_KV has two pinned outputs before its 8 inputs)


if __name__ == "__main__":
    main()
