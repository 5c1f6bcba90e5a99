#!/usr/bin/env python3
"""Generator of the hand-scheduled gfx950 instruction streams of the bf16 dq kernel (plain score).
Writes bwd_dq_tile.inc: string-literal macros that bwd_dq_bf16.hip places inside `asm volatile`
statements: the run loop over steps of two 64-row kv tiles, and prologue / epilogue register moves.

A wave owns 32 q rows (Q^T, dO^T fragments and the dq^T accumulators stay in accumulation
registers); one step covers 128 kv rows = four 32-row kv blocks c = 0..3, software-pipelined:

    A(c): S'^T = K Q^T - lse, dP'^T = V dO^T - delta  16 MFMAs, operands: 16 ds_read_b128 (rows of K, V)
          (Q arrives multiplied by sm_scale log2 e; -lse and -delta enter through the accumulator
          input of each chain's first MFMA, so S' is already the exponent)
    E(c): dS^T = exp2(S'^T) dP'^T            40 VALU ops
    B(c): dq^T += K^T dS^T                  8 MFMAs, operands: 16 ds_read_b64_tr_b16 (K again)

    MFMA order:  A0 | A1 | A2 B0 | A3 B1 | B2 | B3      VALU:  - | E0 | E1 | E2 | E3 | -

LDS reads are issued PREFETCH MFMA pairs ahead of their use into a rotating pool of staging
registers; the next step's K / V tiles are copied global -> LDS by 16 loads spread over the stream.
The emitter (gfx950_stream.py) inserts the s_nop / s_waitcnt that the hardware hazards require.

Register contract with the C++ side (every asm statement names the accumulation registers with
physical-register constraints):
    a[0:63]   dq^T accumulators (4 x 16)   a[64:95] Q^T fragments (8 x 4), pre-scaled   a[96:127] dO^T fragments
    a[128:191] staging slots of the LDS fragments (clobbered)
    v[66:183], s[60:100], vcc, m0   scratch of the run loop (clobbered)
    (the table also names the next work item's first step, copied into LDS during this item's last step)
    %[r0..r7]  byte address of the lane's row fragment ks in K half-tile 0 of the current buffer
    %[t0..t7]  byte address of the lane's transposed fragment (2 db + hi) in K half-tile 0
    %[lse], %[dl]  the lane's q row: log2-domain logsumexp and delta
    %[g0], %[g1v], %[g2], %[g3]  the lane's byte offsets inside a global half tile for the wave's 1 KB blocks
    %[m0], %[m1]  (partial steps) the lane's keep bits: bit 16 (c & 1) + e of m[c >> 1] is element e
               of the S^T accumulator of kv block c; dropped elements get dS = 0
    %[tbl]     LDS byte address of the wave's table of work-group constants (TABLE below)
    %[it], %[kba1], %[kbb1], %[buf]  loop state (in/out); %[it_end] (in); %[partial] (in): the step of the
               run that is partial and takes the masked stream with the keep bits (-1: none)
LDS layout of one step buffer (bytes): K tile 0, K tile 1, V tile 0, V tile 1 (16 KiB each); the two
buffers are 64 KiB apart and the first starts at LDS address 0.
"""
import argparse
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from gfx950_stream import Emitter, Op, address_flips, ar, aset, schedule, vr, vset  # noqa: E402

NSLOT = 8        # staging slots of 8 registers
MIN_AHEAD = 3    # MFMA pairs at least between the LDS reads of a pair and its MFMAs
WAIT_OLD = 20    # a wait for LDS data also covers younger reads issued at least this many instructions ago
CAP = 6          # instructions the scheduler puts between two MFMAs unless deadlines force more
LOAD_FIRST = 0   # MFMA gap from which the first LDS-direct load of the next step may go out
LOAD_EVERY = 3   # gaps between two of them
LOAD_COST = 3    # share of an MFMA gap one of them takes
TRANS_COST = 2   # share of an MFMA gap a transcendental takes (it holds the wave's issue for two slots)
CAP_SOFTCAP = 8  # instructions per MFMA gap in the softcap variant (8 VALU ops per element instead of 2)
S_K2 = "s62"     # (softcap variant) -2 cap log2(e): the table's c2 entry
DROP = ()        # instruction classes left out (--drop, timing studies only)

TILE = 16384
# No scalar operands: constants come from a per-wave table in LDS, loop state from VGPR operands
# (the compiler may print a VGPR for an "s" operand once many uniform values are live).
TABLE = ["n_tiles", "w4k", "c2", "n_steps",  # (c2: softcap and exact-scale variants; its register holds a tile index in the position-bias variant)
         "idx_lo", "idx_hi", "kg_lo", "kg_hi", "vg_lo", "vg_hi", "kban", "kbbn",
         "kgn_lo", "kgn_hi", "vgn_lo", "vgn_hi"]
SREG = {"n_tiles": "s60", "w4k": "s61", "c2": "s62", "n_steps": "s63", "idx_lo": "s64", "idx_hi": "s65",
        "kg_lo": "s66", "kg_hi": "s67", "vg_lo": "s68", "vg_hi": "s69", "kban": "s70", "kbbn": "s71",
        "kgn_lo": "s78", "kgn_hi": "s79", "vgn_lo": "s80", "vgn_hi": "s81",
        "it": "s72", "kba1": "s73", "kbb1": "s74", "buf": "s75", "it_end": "s76", "partial": "s77",
        "idx": "s[64:65]"}
S_SEL = ["s82", "s83", "s96", "s97", "s98", "s99"]  # this pass's tile indices and K / V bases (next step or next item)
STATE_IO = ["it", "kba1", "kbb1", "buf"]
STATE_IN = ["it_end", "partial"]
S_T = ["s84", "s85", "s86", "s87"]
S_GK0, S_GK1, S_GV0, S_GV1 = "s[88:89]", "s[90:91]", "s[92:93]", "s[94:95]"
S_LDSN = "s100"
V_KB2 = 66       # kv tile indices of the step after the next one (2 registers), across the stream
V_TMP = 68       # 4 temporaries of the masked variant
V_TBL = 72       # 12 scratch VGPRs the table is read into at entry
V_S = [72, 104]
V_DP = [88, 120]
V_DS = 136       # dS^T as MFMA B operands: [c & 1][u] x 4 registers
V_NL = 152       # -lse of the lane's q row, 16 copies: accumulator input of the first MFMA of an S chain
V_ND = 168       # -delta of the lane's q row, 16 copies: accumulator input of the first MFMA of a dP chain
V_END = 183
# Position-bias variant (score + slope (j - i)): the accumulator input of a block's S chain,
# slope' (j - i) - lse with slope' = slope log2(e), is itself a matrix product, [1, r] x [b; slope'] with r the
# key's row in the block and b = slope' (j0 - i) - lse for the block's first key j0: one fp32 MFMA per
# block writes it into the registers that hold -lse in the plain variant.
#   %[aone]  A operand: 1.0 in lanes 0-31, float(lane - 32) in lanes 32-63
#   %[mulv]  slope' in lanes 0-31, 0 in lanes 32-63;  %[addv]  -lse of the lane's q row resp. slope'
#   %[iq]    the lane's q index;  %[ka0], %[kb0]  kv tiles of the run's first step
V_B = [184, 185]  # B operands (alternating), 186: a temporary
V_T = 186
V_END_ALIBI = 186
S_CUR = ["s62", "s101"]  # kv tiles of the current step
A_DQ, A_Q, A_DO, A_STG = 0, 64, 96, 128


def bias_ops(e, block, tile, odd):
    """The accumulator input of S chain `block` (its parity picks the B register) for the 32 keys from
    64 `tile` + 32 `odd` on."""
    t0 = S_T[0]
    b = V_B[block & 1]
    e.raw(f"s_lshl_b32 {t0}, {tile}, 6")
    if odd:
        e.raw(f"s_add_u32 {t0}, {t0}, 32")
    e.valu(f"v_sub_u32_e32 {vr(V_T)}, {t0}, %[iq]", vset(V_T), set())
    e.valu(f"v_cvt_f32_i32_e32 {vr(V_T)}, {vr(V_T)}", vset(V_T), vset(V_T))
    e.valu(f"v_fma_f32 {vr(b)}, %[mulv], {vr(V_T)}, %[addv]", vset(b), vset(V_T))
    e.mfma_f32x2(vr(V_NL, 16), "%[aone]", vr(b), vset(V_NL, 16), set(), vset(b))


def build(masked, alibi=False, softcap=False, exact=False):
    em = Emitter()
    em.wait_old = WAIT_OLD
    pairs = []

    def add_A(c):
        for ks in range(8):
            pairs.append(("A", c, ks))

    def add_B(c):
        for u in range(2):
            for j in range(2):
                pairs.append(("B", c, (u, j)))

    add_A(0); add_A(1); add_A(2); add_B(0); add_A(3); add_B(1); add_B(2); add_B(3)
    idx = {key: 2 * k for k, key in enumerate(pairs)}  # number of the pair's first MFMA
    first_A = {c: idx[("A", c, 0)] for c in range(4)}
    last_A = {c: idx[("A", c, 7)] + 1 for c in range(4)}
    first_B = {(c, u): idx[("B", c, (u, 0))] for c in range(4) for u in range(2)}
    last_B = {(c, u): idx[("B", c, (u, 1))] + 1 for c in range(4) for u in range(2)}

    def half_off(c):
        return (c >> 1) * TILE + (c & 1) * (TILE // 2)

    def pair_loads(k):
        kind, c, x = pairs[k]
        base = A_STG + 8 * (k % NSLOT)
        if kind == "A":
            ks = x
            return [(f"ds_read_b128 {ar(base, 4)}, %[r{ks}] offset:{half_off(c)}", aset(base, 4)),
                    (f"ds_read_b128 {ar(base + 4, 4)}, %[r{ks}] offset:{2 * TILE + half_off(c)}", aset(base + 4, 4))]
        u, j = x
        off = half_off(c) + u * 4096
        loads = []
        for i, db in enumerate((2 * j, 2 * j + 1)):
            for hi in range(2):
                reg = base + 4 * i + 2 * hi
                loads.append((f"ds_read_b64_tr_b16 {ar(reg, 2)}, %[t{2 * db + hi}] offset:{off}", aset(reg, 2)))
        return loads

    def pair_mfmas(k):
        kind, c, x = pairs[k]
        base = A_STG + 8 * (k % NSLOT)
        if kind == "A":
            ks = x
            s, dp = V_S[c & 1], V_DP[c & 1]
            cin = V_NL if ks == 0 else s
            cdn = V_ND if ks == 0 else dp
            first = (vr(s, 16), ar(base, 4), ar(A_Q + 4 * ks, 4), vr(cin, 16), vset(s, 16), aset(base, 4), aset(A_Q + 4 * ks, 4),
                     vset(cin, 16))
            if (softcap or exact) and ks == 0:   # (softcap: the chain's result is the exponent of e^(2 s / cap), nothing to
                # start from; exact scale: the raw product, scaled and shifted by one fma per element below)
                first = (vr(s, 16), ar(base, 4), ar(A_Q + 4 * ks, 4), "0", vset(s, 16), aset(base, 4), aset(A_Q + 4 * ks, 4), set())
            return [first,
                    (vr(dp, 16), ar(base + 4, 4), ar(A_DO + 4 * ks, 4), vr(cdn, 16), vset(dp, 16), aset(base + 4, 4),
                     aset(A_DO + 4 * ks, 4), vset(cdn, 16))]
        u, j = x
        ds = V_DS + 8 * (c & 1) + 4 * u
        out = []
        for i, db in enumerate((2 * j, 2 * j + 1)):
            acc = A_DQ + 16 * db
            out.append((ar(acc, 16), ar(base + 4 * i, 4), vr(ds, 4), ar(acc, 16), aset(acc, 16), aset(base + 4 * i, 4),
                        vset(ds, 4), aset(acc, 16)))
        return out

    mfmas = [pair_mfmas(k)[j] for k in range(len(pairs)) for j in range(2)]
    if "mfma" in DROP:
        mfmas = [(lambda e: None)] * len(mfmas)

    def valu(text, dst, src, trans=False, **kw):
        return Op((lambda e: e.valu(text, dst, src, trans)) if "valu" not in DROP else (lambda e: None),
                  cost=TRANS_COST if trans else 1, **kw)

    chains = []
    # ---- E(c): element-wise work between the block's S / dP chains and its B product ----------
    for c in range(4):
        s, dp = V_S[c & 1], V_DP[c & 1]
        ops = []
        for g in range(4):
            if exact:
                # exponent = c2 <q, k> - lse from the raw product: Q went in unscaled, so the logit carries no rounding
                # of a pre-scaled operand (calls whose scale is too large to fold into bf16 Q, see folded_scale_ok)
                for u in range(4):
                    e = 4 * g + u
                    ops.append(valu(f"v_fma_f32 {vr(s + e)}, {vr(s + e)}, {S_K2}, -%[lse]", vset(s + e), vset(s + e) | {("op", "lse")}))
            for u in range(4):
                e = 4 * g + u
                ops.append(valu(f"v_exp_f32_e32 {vr(s + e)}, {vr(s + e)}", vset(s + e), vset(s + e), True))
            if softcap:
                # the chain gave u with e^(2 s / cap) = 2^u:  r = 1 / (2^u + 1), tanh = 1 - 2 r;  dP' r (1 - r) (the
                # derivative's factor 4 goes into the epilogue's scale);  exponent (cap' - lse) - 2 cap' r -> P
                kl = {("op", "lse")}
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
                    ops.append(valu(f"v_fma_f32 {vr(s + e)}, {vr(s + e)}, {S_K2}, %[lse]", vset(s + e), vset(s + e) | kl))
                for u in range(4):
                    e = 4 * g + u
                    ops.append(valu(f"v_exp_f32_e32 {vr(s + e)}, {vr(s + e)}", vset(s + e), vset(s + e), True))
            if masked:
                for u in range(4):
                    e = 4 * g + u
                    ops.append(valu(f"v_bfe_i32 {vr(V_TMP + u)}, %[m{c >> 1}], {16 * (c & 1) + e}, 1", vset(V_TMP + u), set()))
                for u in range(4):
                    e = 4 * g + u
                    ops.append(valu(f"v_and_b32_e32 {vr(s + e)}, {vr(s + e)}, {vr(V_TMP + u)}", vset(s + e), vset(s + e) | vset(V_TMP + u)))
            for u in range(4):
                e = 4 * g + u
                ops.append(valu(f"v_mul_f32_e32 {vr(dp + e)}, {vr(s + e)}, {vr(dp + e)}", vset(dp + e), vset(dp + e) | vset(s + e)))
            # dS^T operand u2 = g >> 1: the registers are those of block c - 2, whose B MFMAs that read
            # them must have been issued; this block's B MFMAs of half u2 wait for them
            u2 = g >> 1
            ds = V_DS + 8 * (c & 1) + 4 * u2 + 2 * (g & 1)
            war = last_B[(c - 2, u2)] + 1 if c >= 2 else 0
            for h in range(2):
                e = 4 * g + 2 * h
                ops.append(valu(f"v_cvt_pk_bf16_f32 {vr(ds + h)}, {vr(dp + e)}, {vr(dp + e + 1)}", vset(ds + h), vset(dp + e, 2),
                                earliest=war, deadline=first_B[(c, u2)] - 1))
        ops[0].earliest = last_A[c] + 4            # the chains' last results need 12 wait states
        if c + 2 < 4:
            ops[-1].deadline = min(ops[-1].deadline, first_A[c + 2])  # A(c + 2) writes the same S / dP registers
        chains.append(ops)

    # ---- LDS reads of the MFMA pairs, in the order of their use: not before the pair that had the
    # staging slot has been issued, at least MIN_AHEAD pairs before their own
    reads = []
    read_texts = []
    for k in range(len(pairs)):
        for text, dst in pair_loads(k):
            reads.append(Op((lambda e, t=text, d=dst: e.lds_read(t, d)) if "lds" not in DROP else (lambda e: None),
                            earliest=max(0, 2 * (k - NSLOT) + 2), deadline=max(0, 2 * (k - MIN_AHEAD))))
            read_texts.append((text, max(0, 2 * (k - MIN_AHEAD))))
    chains.append(reads)
    # the operand addresses move to the other step buffer behind their last read of the step
    chains.append(address_flips(read_texts, lambda name, at: valu(
        f"v_xor_b32_e32 %[{name}], 0x10000, %[{name}]", {("op", name)}, {("op", name)}, earliest=at)))

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

    if alibi:
        # block c's input: behind the first MFMA of A(c - 1), which reads the registers, and 20 wait
        # states before the first one of A(c); block 0 of the next step at the end (its tiles: S_SEL)
        bias = []
        for c in (1, 2, 3, 4):
            tile = S_SEL[0] if c == 4 else S_CUR[c >> 1]
            bias.append(Op(lambda e, c=c, tile=tile: bias_ops(e, c, tile, c & 1), cost=CAP, earliest=first_A[c - 1] + 1,
                           deadline=first_A[c] - 6 if c < 4 else None))
        chains.append(bias)

    schedule(em, mfmas, chains, CAP_SOFTCAP if softcap else CAP)
    em.drain()
    return em


def run_loop(full, masked, alibi=False, softcap=False, exact=False):
    """One asm statement: a run of consecutive steps [it, it_end) of one work item, at most one of
    them partial.  At entry the step's K / V tiles are resident in LDS buffer %[buf]; each pass
    computes the next step's addresses, streams the step (which copies the next step's tiles into the
    other buffer), synchronises the work-group and advances."""
    t0, t1, t2, t3 = S_T
    S = SREG
    n_tbl = len(TABLE)
    entry = [f"ds_read_b128 {vr(V_TBL + 4 * i, 4)}, %[tbl] offset:{16 * i}" for i in range(n_tbl // 4)]
    entry += ["s_waitcnt lgkmcnt(0)"]  # (the streams count LDS operations from zero)
    entry += [f"v_readfirstlane_b32 {S[n]}, {vr(V_TBL + i)}" for i, n in enumerate(TABLE)]
    entry += [f"v_readfirstlane_b32 {S[n]}, %[{n}]" for n in STATE_IO + STATE_IN]
    if alibi:
        pre = Emitter()
        entry += [f"v_readfirstlane_b32 {S_CUR[0]}, %[ka0]", f"v_readfirstlane_b32 {S_CUR[1]}, %[kb0]"]
        bias_ops(pre, 0, S_CUR[0], 0)   # (used by the first MFMA of the loop, more than 20 instructions on)
        entry += pre.out
    elif not softcap and not exact:   # (softcap: %[lse] is cap' - lse and joins the exponent element by element; exact: lse)
        entry += [f"v_sub_f32_e32 {vr(V_NL + e)}, 0, %[lse]" for e in range(16)]
    entry += [f"v_sub_f32_e32 {vr(V_ND + e)}, 0, %[dl]" for e in range(16)]
    top = entry + [".Lfa_dq_loop_%=:"]
    # On the item's last step the tiles copied "for the next step" are the first step of the next
    # work item (its kv tiles and K / V bases come from the table; with no next item they repeat
    # this one's): the next item then starts without waiting for memory.
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
    top += [
        f"s_xor_b32 {t1}, {S['buf']}, 1",
        f"s_lshl_b32 {t1}, {t1}, 16",
        f"s_add_u32 {S_LDSN}, {t1}, {S['w4k']}",
        f"s_mov_b32 m0, {S_LDSN}",   # LDS destination of the step's first copy (the streams write the others)
        # list entries of the step after the next one, clamped into the list: a second half past its
        # end repeats the last tile (finite data; its keep bits are zero)
        f"s_add_u32 {t0}, {S['it']}, 2",
        f"s_lshl_b32 {t0}, {t0}, 1",
        f"s_sub_u32 {t1}, {S['n_tiles']}, 1",
        f"s_min_u32 {t2}, {t0}, {t1}",
        f"s_add_u32 {t0}, {t0}, 1",
        f"s_min_u32 {t3}, {t0}, {t1}",
        f"s_lshl_b32 {t2}, {t2}, 2",
        f"s_lshl_b32 {t3}, {t3}, 2",
        f"v_mov_b32_e32 {vr(V_KB2)}, {t2}",
        f"v_mov_b32_e32 {vr(V_KB2 + 1)}, {t3}",
        f"global_load_dword {vr(V_KB2)}, {vr(V_KB2)}, {S['idx']}",
        f"global_load_dword {vr(V_KB2 + 1)}, {vr(V_KB2 + 1)}, {S['idx']}",
        f"s_cmp_lg_u32 {S['it']}, {S['partial']}",
        "s_cbranch_scc1 .Lfa_dq_full_%=",
    ]
    tail = [
        ".Lfa_dq_tail_%=:",
        "s_waitcnt vmcnt(0) lgkmcnt(0)",
        "s_barrier",
        f"s_add_u32 {S['it']}, {S['it']}, 1",
        f"v_readfirstlane_b32 {S['kba1']}, {vr(V_KB2)}",
        f"v_readfirstlane_b32 {S['kbb1']}, {vr(V_KB2 + 1)}",
        f"s_xor_b32 {S['buf']}, {S['buf']}, 1",
    ]
    if alibi:
        tail += [f"s_mov_b32 {S_CUR[0]}, {ka}", f"s_mov_b32 {S_CUR[1]}, {kb_}"]
    tail += [f"s_cmp_lt_u32 {S['it']}, {S['it_end']}", "s_cbranch_scc1 .Lfa_dq_loop_%="]
    tail += [f"v_mov_b32_e32 %[{n}], {S[n]}" for n in STATE_IO]
    return top + masked.out + ["s_branch .Lfa_dq_tail_%=", ".Lfa_dq_full_%=:"] + full.out + tail


def main():
    global DROP
    here = os.path.dirname(os.path.abspath(__file__))
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("out", nargs="?", default=os.path.join(here, "bwd_dq_tile.inc"))
    ap.add_argument("--drop", default="", help="comma list of mfma,valu,lds,vmem: leave these instruction classes out "
                    "(the stream then computes nothing useful; for timing what bounds it)")
    args = ap.parse_args()
    if args.drop:
        DROP = tuple(x for x in args.drop.split(",") if x)
    with open(args.out, "w") as f:
        f.write("// Generated by gen_dq_tile.py; do not edit.\n")

        def macro(name, lines):
            f.write(f"#define {name} \\\n")
            f.write(" \\\n".join(f'  "{line}\\n"' for line in lines))
            f.write("\n\n")

        full, masked = build(False), build(True)
        macro("FA_DQ_RUN", run_loop(full, masked))
        macro("FA_DQ_RUN_ALIBI", run_loop(build(False, True), build(True, True), True))
        macro("FA_DQ_RUN_SOFTCAP", run_loop(build(False, softcap=True), build(True, softcap=True), softcap=True))
        macro("FA_DQ_RUN_EXACT", run_loop(build(False, exact=True), build(True, exact=True), exact=True))
        for name, em in (("full", full), ("masked", masked)):
            print(f"{args.out}: {name}: {len(em.out)} instructions, {em.stats}", file=sys.stderr)
        macro("FA_DQ_ZERO_ACC", [f"v_accvgpr_write_b32 a{A_DQ + i}, 0" for i in range(64)])
        # Q^T / dO^T fragment ks from 8 dword operands (two pinned outputs come first)
        for ks in range(8):
            macro(f"FA_DQ_PUT_{ks}",
                  [f"v_accvgpr_write_b32 a{A_Q + 4 * ks + i}, %{2 + i}" for i in range(4)]
                  + [f"v_accvgpr_write_b32 a{A_DO + 4 * ks + i}, %{6 + i}" for i in range(4)])
        # accumulator tile t into 16 dword operands; the s_nop of the first one covers the MFMA -> read hazard
        for t in range(4):
            macro(f"FA_DQ_GET_ACC_{t}", (["s_nop 15"] if t == 0 else []) + [f"v_accvgpr_read_b32 %{i}, a{A_DQ + 16 * t + i}" for i in range(16)])


if __name__ == "__main__":
    main()
