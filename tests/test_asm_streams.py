"""Checks of the generated gfx950 instruction streams that need no GPU.

The generators declare, next to every instruction's text, the registers it reads and writes; the
emitter derives s_nop / s_waitcnt from those declarations.  Here the emitted TEXT is parsed again,
registers and all, and the hazard distances are re-derived from the text alone, so a declaration
that does not match its instruction (a wrong register number, a forgotten operand) fails.
"""
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "flex_attention_tpu_amd", "csrc")
sys.path.insert(0, CSRC)

REG = re.compile(r"\b([va])(?:\[(\d+):(\d+)\]|(\d+))")


def regs_of(token):
    out = set()
    for m in REG.finditer(token):
        if m.group(4) is not None:
            out.add((m.group(1), int(m.group(4))))
        else:
            out.update((m.group(1), i) for i in range(int(m.group(2)), int(m.group(3)) + 1))
    return out


def split_operands(line):
    op, _, rest = line.partition(" ")
    rest = re.sub(r"offset:-?\d+", "", rest)
    return op, [t.strip() for t in rest.split(",")] if rest.strip() else []


def check_stream(lines):
    """Replays a stream; returns the number of instructions checked."""
    t = 0
    mfma_w, valu_w, trans_w, dot_w, c_read = {}, {}, {}, {}, {}
    slow = set()  # registers whose MFMA result came from a 16-pass fp32 MFMA: 20 wait states instead of 12
    tracked = (mfma_w, valu_w, trans_w, dot_w, c_read)
    fifo = []  # outstanding LDS reads: destination register sets, oldest first
    skips = {}  # label -> (time behind the forward branch, copies of the tracked maps, LDS queue length)
    n = 0

    def gap(t_def):
        return t - t_def - 1

    def mfma_done(r):
        return r not in mfma_w or gap(mfma_w[r]) >= (20 if r in slow else 12)

    def lds_pending(regs):
        return any(dst & regs for dst in fifo)

    for line in lines:
        op, ops = split_operands(line)
        if op == "s_nop":
            t += int(ops[0]) + 1
            continue
        if op == "s_waitcnt":
            m = re.search(r"lgkmcnt\((\d+)\)", line)
            if m and len(fifo) > int(m.group(1)):
                del fifo[: len(fifo) - int(m.group(1))]
            t += 1
            continue
        if op.endswith(":"):
            # A label that a forward branch of the stream jumps to: what follows must hold both after
            # the skipped block (executed) and without it (no time passed, older writes still there).
            if op[:-1] in skips:
                t0, saved, n_fifo = skips.pop(op[:-1])
                assert len(fifo) == n_fifo, f"LDS traffic inside a skippable block: {line}"
                for cur, old in zip(tracked, saved):
                    merged = dict(old)
                    for r, tw in cur.items():
                        merged[r] = max(merged.get(r, -1 << 30), min(tw, t0 - 1))
                    cur.clear()
                    cur.update(merged)
                t = t0
            continue
        if op.startswith("s_cbranch"):
            t += 1
            label = ops[0]
            if any(l.strip() == label + ":" for l in lines[lines.index(line) + 1:]):
                skips[label] = (t, [dict(d) for d in tracked], len(fifo))
            continue
        if op.startswith("s_"):
            t += 1
            continue
        n += 1
        if op.startswith("v_mfma"):
            assert op in ("v_mfma_f32_32x32x16_bf16", "v_mfma_f32_32x32x2_f32"), line
            dst, a, b, c = (regs_of(x) for x in ops)
            assert not lds_pending(dst | a | b | c), f"MFMA uses a register with an LDS read in flight: {line}"
            for r in a | b:
                assert mfma_done(r), f"MFMA result used as A/B too early: {line}"
            for r in a | b | c | dst:
                assert r not in valu_w or gap(valu_w[r]) >= 2, f"VALU result used by MFMA too early: {line}"
            for r in c - dst:
                assert mfma_done(r), f"MFMA result used as C of another chain too early: {line}"
                c_read[r] = t
            for r in dst:
                mfma_w[r] = t
                (slow.add if op.endswith("_f32") else slow.discard)(r)
                valu_w.pop(r, None)
                trans_w.pop(r, None)
        elif op.startswith("ds_read"):
            dst = regs_of(ops[0])
            assert not lds_pending(dst), f"LDS read into registers of an older read in flight: {line}"
            for r in dst:
                assert mfma_done(r), f"LDS read overwrites a fresh MFMA result: {line}"
                mfma_w.pop(r, None)
                valu_w.pop(r, None)
                trans_w.pop(r, None)
            fifo.append(dst)
        elif op.startswith("global_load_lds"):
            pass  # operands come from the compiler; the destination is LDS through M0
        elif op.startswith("global_store"):
            src = regs_of(ops[1])  # (the address operands come from the compiler and the run loop)
            assert not lds_pending(src), f"store of a register with an LDS read in flight: {line}"
            for r in src:
                assert mfma_done(r), f"store of a fresh MFMA result: {line}"
        elif op.startswith("ds_write"):
            src = regs_of(ops[1])
            assert not lds_pending(src), f"LDS store of a register with an LDS read in flight: {line}"
            fifo.append(set())
        elif op.startswith("v_"):
            dst = regs_of(ops[0])
            src = set().union(*[regs_of(x) for x in ops[1:]]) if len(ops) > 1 else set()
            assert not lds_pending(dst | src), f"VALU uses a register with an LDS read in flight: {line}"
            for r in dst | src:
                assert mfma_done(r), f"VALU touches a fresh MFMA result: {line}"
            for r in src:
                assert r not in trans_w or gap(trans_w[r]) >= 1, f"VALU reads a fresh transcendental result: {line}"
            is_dot = op.startswith("v_dot2c")  # accumulates into its destination
            for r in dst | src:
                if r in dot_w and not (is_dot and r in dst):
                    assert gap(dot_w[r]) >= 3, f"VALU uses a fresh dot-product result: {line}"
            for r in dst:
                assert r not in c_read or gap(c_read.pop(r)) >= 12, f"VALU overwrites the C input of an MFMA in flight: {line}"
                if is_dot:
                    dot_w[r] = t
                else:
                    dot_w.pop(r, None)
            for r in dst:
                mfma_w.pop(r, None)
                valu_w[r] = t
                if op.startswith("v_exp") or op.startswith("v_rcp") or op.startswith("v_log"):
                    trans_w[r] = t
                else:
                    trans_w.pop(r, None)
        else:
            raise AssertionError(f"unknown instruction in stream: {line}")
        t += 1
    assert not fifo, "stream ends with LDS reads in flight"
    assert not skips, f"forward branch to a label that never came: {list(skips)}"
    return n


def scratch_ok(lines, lo, hi, agpr_hi):
    """Every VGPR a stream names lies in its declared scratch range, every AGPR in the pinned range."""
    for line in lines:
        for kind, i in regs_of(line):
            if kind == "v":
                assert lo <= i <= hi, f"v{i} outside the stream's scratch range: {line}"
            else:
                assert 0 <= i <= agpr_hi, f"a{i} outside the pinned range: {line}"


def test_dkv_tile_streams_respect_hazards():
    import gen_dkv_tile as g

    for masked in (False, True):
        em = g.build(masked)
        n = check_stream(em.out)
        assert em.stats["mfma"] == 128  # 4 q blocks x (8 S + 8 dP + 8 dv + 8 dk)
        assert n == em.stats["mfma"] + em.stats["valu"] + em.stats["lds"] + em.stats["vmem"]
        scratch_ok(em.out, 68, 199, 255)
        # position-bias and softcap variants (the latter: 8 element-wise operations per score instead of 2)
        for alibi, softcap in ((True, False), (False, True)):
            v = g.build(masked, alibi, softcap)
            nv = check_stream(v.out)
            assert v.stats["mfma"] == 128
            assert nv == v.stats["mfma"] + v.stats["valu"] + v.stats["lds"] + v.stats["vmem"]
            scratch_ok(v.out, 68, 199, 255)


def test_dkv_export_streams_store_the_dk_operand_and_count_their_waits():
    """dS export variants of the dk/dv streams: every (q block, half) is stored once, from the registers its
    conversions wrote last; the wait of the row values' turn-around counts every vector-memory operation in front
    of it (the two row loads precede the stream), the closing wait the stores behind the last LDS-direct copy."""
    import gen_dkv_tile as g

    for softcap in (False, True):
        for masked in (False, True):
            em = g.build(masked, False, softcap, True)
            n = check_stream(em.out)
            assert em.stats["mfma"] == 128 and em.stats["vmem"] == 24
            assert n == em.stats["mfma"] + em.stats["valu"] + em.stats["lds"] + em.stats["vmem"]
            scratch_ok(em.out, 68, 199, 255)
            last_writer, offsets, vmem, waits, last_load = {}, [], 0, [], -1
            for i, line in enumerate(em.out):
                op, ops = split_operands(line)
                if op.startswith("global_store"):
                    assert op == "global_store_dwordx4" and ops[0] == "%[dsv]" and ops[2] == "s[56:57]", line
                    src = regs_of(ops[1])
                    assert len(src) == 4 and all(last_writer.get(r, "").startswith("v_cvt_pk_bf16_f32") for r in src), line
                    offsets.append(int(re.search(r"offset:(-?\d+)", line).group(1)))
                    vmem += 1
                elif op.startswith("global_load_lds"):
                    vmem += 1
                    last_load = vmem
                elif op == "s_waitcnt" and "vmcnt" in line:
                    waits.append((int(re.search(r"vmcnt\((\d+)\)", line).group(1)), vmem))
                elif op.startswith("v_") and ops:
                    for r in regs_of(ops[0]):
                        last_writer[r] = op
            assert sorted(offsets) == [1024 * k - 4096 for k in range(8)]
            # the stored registers are the B operands of the dk MFMAs (dk accumulators a[64:127])
            dk_b = set()
            for line in em.out:
                op, ops = split_operands(line)
                if op.startswith("v_mfma") and regs_of(ops[0]) <= {("a", i) for i in range(64, 128)}:
                    dk_b |= regs_of(ops[2])
            stored = set()
            for line in em.out:
                op, ops = split_operands(line)
                if op.startswith("global_store"):
                    stored |= regs_of(ops[1])
            assert stored == dk_b
            assert len(waits) == 2
            (n_turn, at_turn), (n_end, at_end) = waits
            assert n_turn == at_turn, "the turn-around must wait for exactly the operations in front of it"
            assert at_end == vmem == 24 and n_end == vmem - last_load, "the closing wait leaves only stores behind the last copy open"


def test_hazard_checker_catches_a_bad_stream():
    bad = ["v_mfma_f32_32x32x16_bf16 v[72:87], v[192:195], a[128:131], 0", "v_exp_f32_e32 v72, v72"]
    with pytest.raises(AssertionError):
        check_stream(bad)
    bad = ["ds_read_b128 v[192:195], %[r0] offset:0", "v_mfma_f32_32x32x16_bf16 v[72:87], v[192:195], a[128:131], 0"]
    with pytest.raises(AssertionError):
        check_stream(bad)
    bad = ["v_cvt_pk_bf16_f32 v136, v72, v73", "v_mfma_f32_32x32x16_bf16 a[0:15], v[192:195], v[136:139], a[0:15]"]
    with pytest.raises(AssertionError):
        check_stream(bad)
    # the result of the 16-pass fp32 MFMA as accumulator input of another chain: 20 wait states
    slow = ["v_mfma_f32_32x32x2_f32 v[152:167], v0, v184, 0", "s_nop 15",
            "v_mfma_f32_32x32x16_bf16 v[72:87], a[128:131], a[64:67], v[152:167]"]
    with pytest.raises(AssertionError):
        check_stream(slow)
    check_stream(slow[:2] + ["s_nop 3"] + slow[2:])


def test_generated_include_matches_generator(tmp_path):
    out = tmp_path / "tile.inc"
    subprocess.run([sys.executable, os.path.join(CSRC, "gen_dkv_tile.py"), str(out)], check=True, capture_output=True)
    text = out.read_text()
    for macro in ("FA_DKV_RUN", "FA_DKV_ZERO_ACC", "FA_DKV_PUT_KV_7", "FA_DKV_GET_ACC_7"):
        assert f"#define {macro} " in text


@pytest.mark.skipif(not os.path.exists("/opt/rocm/bin/hipcc"), reason="needs hipcc")
def test_compiler_keeps_out_of_the_pinned_registers(tmp_path):
    """Outside the asm statements the plain-score dk/dv kernel must not touch a[0:191] (the streams'
    accumulators and K/V fragments) and must not spill inside the loop over an item's runs (loop depth 2 and
    deeper): both would mean the compiler moved the pinned state around the statements.  At the level of the
    item loop a few spilled dwords of long-lived values are tolerated (one store in front of the loop and one
    reload per item today)."""
    from flex_attention_tpu_amd import build as B

    gen = tmp_path / "bwd_dkv_tile.inc"
    subprocess.run([sys.executable, os.path.join(CSRC, "gen_dkv_tile.py"), str(gen)], check=True, capture_output=True)
    asm = tmp_path / "dkv.s"
    flags = [f for f in B.FLAGS if f != "-fPIC"]
    r = subprocess.run([B.HIPCC, *flags, f"-I{tmp_path}", "-S", "--cuda-device-only", os.path.join(CSRC, "bwd_dkv_bf16.hip"),
                        "-o", str(asm)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    text = asm.read_text().split("\n")
    start = next(i for i, l in enumerate(text) if l.startswith("_ZN2fa30bwd_dkv_bf16_d128_plain_kernelILi0ELb0ELb0E"))  # (plain score, no document ids, no dS export)
    end = next(i for i, l in enumerate(text) if i > start and l.strip() == "s_endpgm")
    in_asm = False
    depth, shallow_spills = 0, 0
    for line in text[start:end]:
        stripped = line.strip()
        if re.match(r"(\.LBB\d+_\d+:|; %bb\.\d+:)", stripped):   # a basic block starts: its comment names the loop depth
            m = re.search(r"Depth=(\d+)", stripped)
            depth = int(m.group(1)) if m else 0
        elif stripped.startswith(";") and "Loop Header: Depth=" in stripped:   # (header comments run over several lines)
            depth = int(re.search(r"Loop Header: Depth=(\d+)", stripped).group(1))
        if "#ASMSTART" in line:
            in_asm = True
        elif "#ASMEND" in line:
            in_asm = False
        elif not in_asm and not stripped.startswith((";", ".")):
            if "scratch_" in line:
                assert depth < 2, f"spill inside the run loop of the plain-score dk/dv kernel: {line}"
                shallow_spills += 1
            for kind, i in regs_of(line.split(";")[0]):
                assert kind != "a", f"compiler touches an accumulation register: {line}"
    assert shallow_spills <= 4, f"{shallow_spills} spill instructions in the plain-score dk/dv kernel"


def test_dq_tile_streams_respect_hazards():
    import gen_dq_tile as g

    for masked in (False, True):
        em = g.build(masked)
        n = check_stream(em.out)
        assert em.stats["mfma"] == 96  # 4 kv blocks x (8 S + 8 dP + 8 dq)
        assert n == em.stats["mfma"] + em.stats["valu"] + em.stats["lds"] + em.stats["vmem"]
        scratch_ok(em.out, 66, 183, 191)
        # position-bias variant: one fp32 MFMA per block more, writing the S chains' accumulator input
        em = g.build(masked, True)
        n = check_stream(em.out)
        assert em.stats["mfma"] == 96 and em.stats["mfma32"] == 4
        assert n == em.stats["mfma"] + em.stats["mfma32"] + em.stats["valu"] + em.stats["lds"] + em.stats["vmem"]
        scratch_ok(em.out, 66, 186, 191)
        # softcap variant: eight element-wise operations per score instead of two, same MFMAs
        em = g.build(masked, softcap=True)
        n = check_stream(em.out)
        assert em.stats["mfma"] == 96
        assert n == em.stats["mfma"] + em.stats["valu"] + em.stats["lds"] + em.stats["vmem"]
        scratch_ok(em.out, 66, 183, 191)
        check_dataflow(em.out, 1, 4)
        # exact-scale variant: Q unscaled, one fma per score turns the raw product into the exponent
        em = g.build(masked, exact=True)
        n = check_stream(em.out)
        assert em.stats["mfma"] == 96 and sum("v_fma_f32" in l for l in em.out) == 64
        assert n == em.stats["mfma"] + em.stats["valu"] + em.stats["lds"] + em.stats["vmem"]
        scratch_ok(em.out, 66, 183, 191)
        check_dataflow(em.out, 1, 4)


def test_fwd_tile_streams_respect_hazards():
    import gen_fwd_tile as g

    for masked in (False, True):
        em = g.build(masked)
        n = check_stream(em.out)
        assert em.stats["mfma"] == 128  # 4 kv blocks x 2 q blocks x (8 S + 8 PV)
        assert n == em.stats["mfma"] + em.stats["valu"] + em.stats["lds"] + em.stats["vmem"]
        scratch_ok(em.out, 66, 199, 255)
        # position-bias variant: one fp32 MFMA per S chain more, writing the chain's accumulator input
        ab = g.build(masked, True)
        nb = check_stream(ab.out)
        assert ab.stats["mfma"] == 128 and ab.stats["mfma32"] == 8
        assert nb == ab.stats["mfma"] + ab.stats["mfma32"] + ab.stats["valu"] + ab.stats["lds"] + ab.stats["vmem"]
        scratch_ok(ab.out, 66, 201, 255)
        # softcap variant: no maximum is tracked, no branch at all, 6.5 element-wise operations per score
        sc = g.build(masked, softcap=True)
        ns = check_stream(sc.out)
        assert sc.stats["mfma"] == 128 and not any(l.startswith(("s_cbranch", "s_branch")) for l in sc.out)
        assert ns == sc.stats["mfma"] + sc.stats["valu"] + sc.stats["lds"] + sc.stats["vmem"]
        scratch_ok(sc.out, 66, 199, 255)
        check_dataflow(sc.out, 2, 4)
        # between a forward branch and its label there is only VALU / scalar work: a skipped MFMA,
        # LDS read or wait would break the stream's bookkeeping
        pending = None
        for line in em.out + ab.out:
            if line.startswith("s_cbranch"):
                pending = line.split()[1]
            elif pending and line.strip() == pending + ":":
                pending = None
            elif pending:
                assert not line.startswith(("v_mfma", "ds_", "global_load", "s_waitcnt")), (pending, line)
        assert pending is None


def check_dataflow(lines, reads_per_fragment, reads_per_packed):
    """What the hazard rules cannot see: that the scheduler kept every value alive until its users
    were issued.  Re-derived from the text alone:
      * a staging register filled by an LDS read is read by exactly `reads_per_fragment` MFMAs (as A
        operand) before the next LDS read overwrites it;
      * a register written by v_cvt_pk_bf16_f32 (P, dS) is read by exactly `reads_per_packed` MFMAs
        (as B operand) before it is packed again;
      * an accumulation chain (first MFMA: C input is not its destination) consists of 8 MFMAs, and
        no other instruction touches its destination before the eighth has been issued."""
    frag_reads, packed_reads, chain = {}, {}, {}
    skip = None
    for line in lines:
        op, ops = split_operands(line)
        if op.startswith("s_cbranch"):
            skip = ops[0]  # the correction blocks only run when needed: not part of the steady flow
            continue
        if skip is not None:
            if line.strip() == skip + ":":
                skip = None
            continue
        if op.startswith("v_mfma"):
            dst, a, b, c = (regs_of(x) for x in ops)
            for r in a:
                if r in frag_reads:
                    frag_reads[r] += 1
            for r in b:
                if r in packed_reads:
                    packed_reads[r] += 1
            if dst and next(iter(dst))[0] == "v":  # S / dP chains live in VGPRs
                key = min(dst)
                if c != dst:
                    assert chain.get(key, 8) == 8, f"a chain restarts after {chain[key]} MFMAs: {line}"
                    chain[key] = 1
                else:
                    chain[key] += 1
                    assert chain[key] <= 8, f"more than 8 MFMAs in a chain: {line}"
        elif op.startswith("ds_read"):
            for r in regs_of(ops[0]):
                if r[0] == "a":
                    assert frag_reads.get(r, reads_per_fragment) == reads_per_fragment, \
                        f"fragment in {r} overwritten after {frag_reads[r]} of {reads_per_fragment} uses: {line}"
                    frag_reads[r] = 0
        elif op.startswith("v_"):
            touched = set().union(*[regs_of(x) for x in ops]) if ops else set()
            for key, n in chain.items():
                tup = {(key[0], key[1] + i) for i in range(16)}
                assert not (touched & tup) or n == 8, f"chain at {key} used after {n} of 8 MFMAs: {line}"
            if op.startswith("v_cvt_pk_bf16"):
                for r in regs_of(ops[0]):
                    assert packed_reads.get(r, reads_per_packed) == reads_per_packed, \
                        f"packed operand {r} rewritten after {packed_reads[r]} of {reads_per_packed} uses: {line}"
                    packed_reads[r] = 0
    # the stream repeats: what is still open at its end is consumed... nothing may be open
    for r, n in frag_reads.items():
        assert n == reads_per_fragment, f"fragment in {r} used {n} times at the end of the stream"
    for r, n in packed_reads.items():
        assert n == reads_per_packed, f"packed operand {r} used {n} times at the end of the stream"
    assert all(n == 8 for n in chain.values())


def test_streams_keep_values_alive_for_their_users():
    import gen_dkv_tile, gen_dq_tile, gen_fwd_tile

    for masked in (False, True):
        # dk/dv, dq: every fragment feeds one MFMA, every packed P / dS register four (d blocks)
        check_dataflow(gen_dkv_tile.build(masked).out, 1, 4)
        check_dataflow(gen_dq_tile.build(masked).out, 1, 4)
        # forward: a K row fragment feeds both q blocks, a V^T fragment likewise
        check_dataflow(gen_fwd_tile.build(masked).out, 2, 4)


def test_dataflow_check_catches_an_early_overwrite():
    import gen_dq_tile

    out = list(gen_dq_tile.build(False).out)
    i = next(k for k, l in enumerate(out) if l.startswith("ds_read_b128 a[136:139]"))
    j = next(k for k in range(i + 1, len(out)) if out[k].startswith("v_mfma") and "a[136:139]" in out[k])
    moved = out[:i] + out[i + 1:j + 1] + [out[i]] + out[j + 1:]  # the read now follows its user
    with pytest.raises(AssertionError):
        check_dataflow(moved, 1, 4)



def test_fwd_out_of_line_blocks_are_the_inline_ones():
    """gen_fwd_tile.out_of_line moves the skipped-unless-needed blocks behind the loop: putting every moved
    block back where its branch is gives the stream the hazard checks above ran on, line for line, and the
    common path that is left holds no branch that is normally taken."""
    import gen_fwd_tile as g
    direct = {"s_cbranch_vccnz": "s_cbranch_vccz", "s_cbranch_scc0": "s_cbranch_scc1"}
    for masked in (False, True):
        lines = g.build(masked).out
        hot, cold = g.out_of_line(lines)
        assert len(hot) + len(cold) == len(lines) + 2 * sum(1 for l in cold if l.startswith("s_branch"))
        blocks = {}
        cur = None
        for l in cold:
            if cur is None:
                assert l.endswith(":")
                cur = l[:-1]
                blocks[cur] = []
            elif l.startswith("s_branch"):
                blocks[cur].append(l.split()[1])  # where it returns to
                cur = None
            else:
                blocks[cur].append(l)
        assert cur is None and len(blocks) == 8    # the blocks that move M (sequential chains need no late corrections)
        back = []
        i = 0
        while i < len(hot):
            parts = hot[i].split()
            if len(parts) == 2 and parts[1] in blocks:
                body = blocks[parts[1]]
                assert hot[i + 1] == body[-1] + ":", "the block returns to the instruction behind its branch"
                back += [f"{direct[parts[0]]} {body[-1]}"] + body[:-1] + [hot[i + 1]]
                i += 2
            else:
                assert not hot[i].startswith(("s_cbranch", "s_branch")), hot[i]
                back.append(hot[i])
                i += 1
        assert back == lines


# ---------------------------------------------------------------------------------------------------
# vector-memory queue of the run loops: no load into registers may be open when control leaves the asm
# ---------------------------------------------------------------------------------------------------
def check_vmem_queue(lines):
    """Walks every control-flow path of an asm region (forward and backward branches, both outcomes of
    every conditional one) and replays the in-order vector-memory queue: loads into VGPRs, LDS-direct
    loads and stores enter it, `s_waitcnt vmcnt(N)` retires all but the N youngest.  Asserts that

      * no instruction names a VGPR that a load still in the queue will write (the value is not there
        yet; and if the compiler or the stream reused the register, the late load would overwrite it);
      * at every `s_barrier` no load of either kind is open (the barrier tells the other waves that
        this wave's copies have landed);
      * where control leaves the region (falls off its end) only stores are open: the compiler, which
        does not know of the region's loads, is free to reuse every register behind it.

    Returns the number of (instruction, queue state) pairs visited."""
    labels = {l[:-1]: i for i, l in enumerate(lines) if l.endswith(":")}
    seen = set()
    work = [(0, ())]
    while work:
        pc, q = work.pop()
        while True:
            if (pc, q) in seen:
                break
            seen.add((pc, q))
            if pc == len(lines):
                open_loads = [e for e in q if e[0] != "store"]
                assert not open_loads, f"region ends with loads in flight: {open_loads}"
                break
            line = lines[pc]
            op, ops = split_operands(line)
            pending = set().union(*[set(e[1]) for e in q]) if q else set()
            if op.endswith(":"):
                pc += 1
                continue
            if op == "s_waitcnt":
                m = re.search(r"vmcnt\((\d+)\)", line)
                if m:
                    n = int(m.group(1))
                    q = q[len(q) - n:] if n < len(q) else q
                    if n == 0:
                        q = ()
                pc += 1
                continue
            if op == "s_barrier":
                open_loads = [e for e in q if e[0] != "store"]
                assert not open_loads, f"s_barrier with loads in flight: {open_loads}"
                pc += 1
                continue
            if op == "s_branch":
                pc = labels[ops[0]]
                continue
            if op.startswith("s_cbranch"):
                work.append((labels[ops[0]], q))
                pc += 1
                continue
            named = regs_of(line)
            assert not (named & pending), f"register of a load in flight is used: {line}"
            if op.startswith("global_load_lds"):
                q = q + (("lds", ()),)
            elif op.startswith("global_load") or op.startswith("buffer_load"):
                q = q + (("load", tuple(sorted(regs_of(ops[0])))),)
            elif op.startswith("global_store") or op.startswith("buffer_store"):
                q = q + (("store", ()),)
            pc += 1
    return len(seen)


def _run_loops():
    import gen_dkv_tile, gen_dq_tile, gen_fwd_tile
    for alibi, softcap, export in ((False, False, False), (True, False, False), (False, True, False), (False, False, True),
                                   (False, True, True)):
        g = gen_dkv_tile
        yield f"dkv alibi={alibi} softcap={softcap} export={export}", g.run_loop(
            g.build(False, alibi, softcap, export), g.build(True, alibi, softcap, export), alibi, softcap, export)
    for g, name in ((gen_dq_tile, "dq"), (gen_fwd_tile, "fwd")):
        for alibi, softcap in ((False, False), (True, False), (False, True)):
            yield f"{name} alibi={alibi} softcap={softcap}", g.run_loop(
                g.build(False, alibi, softcap), g.build(True, alibi, softcap), alibi, softcap)
    yield "dq exact", gen_dq_tile.run_loop(gen_dq_tile.build(False, exact=True), gen_dq_tile.build(True, exact=True), exact=True)


def test_run_loops_leave_no_load_in_flight():
    """Every generated run loop (the dq and dk/dv ones are the only asm regions of the library that load
    from global memory into registers; every other asm load, the forward loop's included, has LDS as its
    destination and is waited for with vmcnt(0) in front of the work-group barrier): on every path through the region the loads into registers have been waited
    for before their registers are named again and before control leaves the region, and all copies into
    LDS before each barrier.  The dS-exporting loops may leave stores open, nothing else."""
    n_loops = 0
    for name, lines in _run_loops():
        # (the check is not vacuous: every loop copies into LDS, the backward loops also load into registers)
        assert any(l.startswith("global_load_lds") for l in lines), name
        assert name.startswith("fwd") or any(l.startswith("global_load_dword") for l in lines), name
        assert check_vmem_queue(lines) > len(lines), name
        n_loops += 1
    assert n_loops == 12


def test_vmem_queue_checker_catches_open_loads():
    # a load into a register that is still open where the region ends
    bad = ["global_load_dword v66, v66, s[66:67]", "v_mov_b32_e32 v70, 0"]
    with pytest.raises(AssertionError, match="ends with loads in flight"):
        check_vmem_queue(bad)
    check_vmem_queue(bad + ["s_waitcnt vmcnt(0)"])
    # ... open on one of two paths only (the wait is skipped by a branch)
    bad = ["global_load_dword v66, v66, s[66:67]", "s_cbranch_scc1 .Lskip", "s_waitcnt vmcnt(0)", ".Lskip:", "s_nop 0"]
    with pytest.raises(AssertionError, match="ends with loads in flight"):
        check_vmem_queue(bad)
    # a store behind the load may stay open, the load may not: vmcnt(1) retires the load, vmcnt(2) does not
    ok = ["global_load_dword v66, v66, s[66:67]", "global_store_dwordx4 v80, v[72:75], s[56:57]", "s_waitcnt vmcnt(1)"]
    check_vmem_queue(ok)
    with pytest.raises(AssertionError, match="ends with loads in flight"):
        check_vmem_queue(ok[:2] + ["s_waitcnt vmcnt(2)"])
    # the destination is read before the wait
    bad = ["global_load_dword v66, v66, s[66:67]", "v_readfirstlane_b32 s80, v66", "s_waitcnt vmcnt(0)"]
    with pytest.raises(AssertionError, match="register of a load in flight"):
        check_vmem_queue(bad)
    # a copy into LDS still open at the barrier, across a loop back-edge
    bad = [".Ltop:", "s_barrier", "global_load_lds_dwordx4 v70, s[20:21]", "s_cbranch_scc1 .Ltop", "s_waitcnt vmcnt(0)"]
    with pytest.raises(AssertionError, match="s_barrier with loads in flight"):
        check_vmem_queue(bad)
