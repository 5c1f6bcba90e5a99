"""Benchmark of the flex-attention hot path on one MI355X.

One step = one pass of the hot path over one batch of synthetic input resident in HBM:
forward (saving l, m), delta pre-pass, dq backward, dk/dv backward (where the package's own backward does so,
softcap scores and masks with many partial tiles, the dk/dv pass hands its dS to the dq pass; where the kernels
can run either way the other way is timed beside it).  The headline workload is
benchmark configurations 2 + 3 (B=4, H=32, S=4096, D=128, bf16, causal); the other configurations
(cfg1 fp32 small, cfg4 ALiBi + causal window, cfg5 GQA + soft-cap + documents; and d256, cfg2's FLOPs at head
dimension 256, which is not one of the reference's configurations) are measured in the
same run and reported as sub-objects (`--config NAME` makes one of them the headline instead).
Prints ONE JSON line: whole-step algorithmic TFLOP/s, per-pass TFLOP/s and fraction of the bf16
MFMA peak, launch-time quantiles, a roofline object for the dominant kernel and the CPU oracle
timed on the host cores.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X published dense bf16 MFMA peak
PEAK_HBM_GBS = 8000.0
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "bench_cfg2_hbm_traffic.txt")


def kernel_sources_digest():
    """sha256 (first 16 hex digits) over the kernel sources of libflexattn.so: the HIP files, their headers and
    the stream generators, in name order.  The counter summary under profiles/ records the digest of the
    sources it was measured on; a different digest here means the kernels changed since."""
    import hashlib
    csrc = os.path.join(ROOT, "flex_attention_tpu_amd", "csrc")
    h = hashlib.sha256()
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".hip", ".hpp", ".py")):
            h.update(name.encode())
            h.update(open(os.path.join(csrc, name), "rb").read())
    return h.hexdigest()[:16]


def counter_traffic(kernel):
    """(HBM bytes per launch of `kernel` on cfg2, stale) from the committed rocprofv3 counter summary
    (FETCH_SIZE and WRITE_SIZE runs of this script, scaled by the 256 MiB device copy main() ends with), or
    (None, None).  Counter-derived in a separate profiler run, not measured in this run: `stale` says whether
    the kernel sources have changed since that run (the summary names the digest it was measured on)."""
    value, digest = None, None
    try:
        for line in open(TRAFFIC_PROFILE):
            f = line.split()
            if len(f) >= 6 and f[0] == kernel and re.fullmatch(r"[0-9.]+", f[5]):
                value = int(float(f[5]) * 1e6)
            m = re.match(r"kernel sources digest: ([0-9a-f]{16})", line)
            if m:
                digest = m.group(1)
    except OSError:
        pass
    if value is None:
        return None, None
    return value, digest != kernel_sources_digest()


def cpu_baseline(cfg, budget_s=12.0):
    """Times the CPU oracle (float32 math on the dtype-rounded inputs) on a bounded sample of the
    same workload: whole (batch, head) pairs of the configuration, forward + backward."""
    import torch
    from oracle import mha_oracle as O
    from flex_attention_tpu_amd import configs
    okw = O.kwargs_for_config(cfg)
    group = cfg.Hq // cfg.Hkv
    q, k, v, do = O.make_inputs(1, group, 1, cfg.S, cfg.S, cfg.D, dtype=cfg.dtype, seed=cfg.seed)
    if "score_mod" in okw and cfg.score == "alibi":
        okw["score_mod"] = O.score_mod_alibi_global(O.alibi_slopes(cfg.Hq)[:group])
    n_done, t_total = 0, 0.0
    kw = dict(sm_scale=cfg.sm_scale, compute_dtype=torch.float32, **okw)
    while True:
        t0 = time.perf_counter()
        o, l, m = O.mha_reference(q, k, v, save_residuals=True, **kw)
        O.mha_bwd_reference(q, k, v, o, do, l, m, **kw)
        t_total += time.perf_counter() - t0
        n_done += 1
        if t_total > budget_s:
            break
    flops_per_group = 3.5 * configs.flops_fwd(cfg) / (cfg.B * cfg.Hkv)
    return {
        "value": flops_per_group * n_done / t_total / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{n_done} x (1 batch, 1 kv head = {group} q head(s)) of {cfg.name} fwd+bwd, fp32 torch-CPU "
                  f"restatement of mha_reference.py, {t_total:.1f} s, host cpu_count={os.cpu_count()}",
    }


def quantiles(xs):
    xs = sorted(xs)
    pick = lambda f: xs[min(len(xs) - 1, int(round(f * (len(xs) - 1))))]
    return {"median": pick(0.5), "p10": pick(0.1), "p90": pick(0.9)}


def measure(cfg, steps, warmup):
    """Wall time of `steps` whole steps and per-kernel launch durations of one configuration."""
    import torch
    import flex_attention_tpu_amd as F
    from flex_attention_tpu_amd import configs
    import warnings

    dev = torch.device("cuda:0")
    q, k, v, do = configs.make_inputs(cfg, dev)
    mf, bf = configs.mask_fns(cfg)
    sfn = configs.score_fn(cfg)
    sc, blk = cfg.sm_scale, cfg.block
    warnings.filterwarnings("ignore", message="score_fn with sm_scale")  # (the configurations use 1/sqrt(D) on purpose)

    def fwd():
        return F._flex_attention_impl(q, k, v, None, None, True, False, sc, 1, blk, blk, blk, False, bf, mf, sfn)

    def dq_of(o, l, m, d, ds=None):
        # d=None: the dq pass takes delta = sum(o * do) itself and returns it next to dq
        return F.flex_attention_bwd_dq(q, k, v, None, None, l, m, o, do, d, block_b=1, block_q=blk, block_k_major=blk,
                                       block_k=blk, sm_scale=sc, debug=False, score_fn=sfn, mask_fn=mf, block_mask_fn=bf,
                                       ds=ds, return_delta=d is None)

    def dkv_of(l, m, d, return_ds=False):
        return F.flash_attention_bwd_dkv(k, v, q, None, None, l, m, d, do, block_b=1, block_q=blk, block_q_major=blk,
                                         block_k_major=blk, block_k=blk, sm_scale=sc, causal=False, debug=False,
                                         score_fn=sfn, mask_fn=mf, block_mask_fn=bf, return_ds=return_ds)

    # the step hands dS over where the package's own backward (flex_attention) would: ds_exchange_pays
    from flex_attention_tpu_amd.flex_attention_dq_bwd import ds_exchange_pays
    exchange = ds_exchange_pays(sfn, mf) and q.dtype == torch.bfloat16

    def step():
        o, l, m = fwd()
        if not exchange:   # delta, dq and dk/dv from one call (flexattn_bwd), as the package's own backward runs them
            return (o,) + F.flex_attention_bwd(q, k, v, None, None, l, m, o, do, block_q=blk, block_k=blk, sm_scale=sc,
                                               score_fn=sfn, mask_fn=mf, block_mask_fn=bf)
        d = F.compute_delta(o, do)
        dk, dv, ds = dkv_of(l, m, d, True)   # (ds is None where the configuration's kernels exchange nothing)
        return o, dq_of(o, l, m, d, ds), dk, dv

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    # Per-kernel launch durations: K back-to-back launches of one kernel between two HIP events on the launch
    # stream give the mean (events around single launches carry several us of marker overhead; the shorter of two
    # such batches is reported); an event
    # behind every launch of a second batch gives the launch-to-launch intervals for the quantiles.
    o, l, m = fwd()
    d = F.compute_delta(o, do)
    ds = dkv_of(l, m, d, True)[2]   # (None where the configuration's kernels exchange nothing)
    used = exchange and ds is not None
    fused = not exchange   # the dq call launches the delta kernel itself (d=None): the step makes no delta call
    launches = {"fwd": fwd, "delta": lambda: F.compute_delta(o, do),
                "dq": (lambda: dq_of(o, l, m, d, ds)) if used else (lambda: dq_of(o, l, m, None if fused else d)),
                "dkv": (lambda: dkv_of(l, m, d, True)) if used else (lambda: dkv_of(l, m, d))}
    if fused:
        launches["dq_given_delta"] = lambda: dq_of(o, l, m, d)   # the dq pass alone, delta from its own launch
    if ds is not None:   # the other way of running the two passes, for comparison
        launches.update(dq_other=(lambda: dq_of(o, l, m, None)) if used else (lambda: dq_of(o, l, m, d, ds)),
                        dkv_other=(lambda: dkv_of(l, m, d)) if used else (lambda: dkv_of(l, m, d, True)))
    ms, quant = {}, {}
    for name, fn in launches.items():
        for _ in range(3):   # (buffers a launch allocates for the first time are slow on first touch)
            fn()
        torch.cuda.synchronize()
        batch = []
        for _ in range(2):   # (two batches, the shorter one counts: a single stalled launch, which these boxes show
            # now and then, otherwise adds its tens of milliseconds to the mean of thirty)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(steps):
                fn()
            e1.record()
            torch.cuda.synchronize()
            batch.append(e0.elapsed_time(e1) / steps)
        ms[name] = min(batch)
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
        fn()
        ev[0].record()
        for i in range(steps):
            fn()
            ev[i + 1].record()
        torch.cuda.synchronize()
        quant[name] = quantiles([ev[i].elapsed_time(ev[i + 1]) for i in range(steps)])
    return {"ms_step": wall * 1e3 / steps, "ms": ms, "quantiles_ms": quant, "elem_bytes": q.element_size(),
            "numel_q": q.numel(), "numel_k": k.numel(), "ds_bytes": ds.buf.numel() if ds is not None else 0,
            "ds_used": used, "delta_fused": fused}


def tf(fl, t_ms):
    return fl / (t_ms * 1e-3) / 1e12


def summary(cfg, r):
    """Per-pass figures of one configuration: ms, TFLOP/s and fraction of the MFMA peak for the bf16
    configurations; microseconds and GB/s of algorithmic traffic for the small fp32 one."""
    from flex_attention_tpu_amd import configs
    ms = r["ms"]
    f_fwd = configs.flops_fwd(cfg)
    fused = r["delta_fused"]   # ms["dq"] is then the dq call that launches the delta kernel and the dq kernel
    ms_bwd = (0.0 if fused else ms["delta"]) + ms["dq"] + ms["dkv"]
    eb, nq, nk = r["elem_bytes"], r["numel_q"], r["numel_k"]
    rows = 4 * cfg.B * cfg.Hq * cfg.S
    bytes_delta = 2 * nq * eb + rows
    out = {
        "workload": f"{cfg.name}: B={cfg.B} Hq={cfg.Hq} Hkv={cfg.Hkv} S={cfg.S} D={cfg.D} "
                    f"{'bf16' if eb == 2 else 'fp32'}, mask={cfg.mask}, score={cfg.score}",
        "ms_per_step": r["ms_step"], "step_tflops": tf(3.5 * f_fwd, r["ms_step"]),
        "fwd": {"ms": ms["fwd"], "tflops": tf(f_fwd, ms["fwd"]), **r["quantiles_ms"]["fwd"]},
        "bwd": {"ms": ms_bwd, "tflops": tf(2.5 * f_fwd, ms_bwd), "delta_ms": ms["delta"], "dq_ms": ms["dq"],
                "dkv_ms": ms["dkv"], "delta_gbs": bytes_delta / (ms["delta"] * 1e-3) / 1e9,
                "dq_quantiles_ms": r["quantiles_ms"]["dq"], "dkv_quantiles_ms": r["quantiles_ms"]["dkv"],
                "delta_quantiles_ms": r["quantiles_ms"]["delta"], "ds_exchange": r["ds_used"],
                "delta_launched_by_dq_call": fused},
    }
    if fused:   # (dq_ms covers the delta kernel and the dq kernel; delta_ms and the dq kernel alone beside it)
        out["bwd"].update(dq_kernel_ms=ms["dq_given_delta"],
                          ms_with_separate_delta_call=ms["delta"] + ms["dq_given_delta"] + ms["dkv"])
    if r["ds_bytes"] > 0:   # the backward run the other way (with the dS hand-over if the step runs without, and vice versa)
        # (the hand-over needs delta before the dk/dv pass: its own launch; the recomputing way takes it in the dq pass)
        ms_other = (0.0 if r["ds_used"] else ms["delta"]) + ms["dq_other"] + ms["dkv_other"]
        tag = "without_exchange" if r["ds_used"] else "with_exchange"
        out["bwd"].update({"ds_buffer_bytes": r["ds_bytes"], f"dq_ms_{tag}": ms["dq_other"], f"dkv_ms_{tag}": ms["dkv_other"],
                           f"ms_{tag}": ms_other, f"tflops_{tag}": tf(2.5 * f_fwd, ms_other)})
    if eb == 2:
        out["fwd"]["frac_of_peak"] = out["fwd"]["tflops"] / PEAK_BF16_TFLOPS
        out["bwd"]["frac_of_peak"] = out["bwd"]["tflops"] / PEAK_BF16_TFLOPS
    else:
        # launch/latency-bound fp32 case: time per pass and algorithmic GB/s (warm caches: 2 MB of operands)
        b_fwd = (nq + 2 * nk + nq) * eb + 2 * rows                  # q, k, v in; o, l, m out
        b_dq = (2 * nq + 2 * nk) * eb + 3 * rows + nq * eb           # q, do, k, v, l, m, delta in; dq out
        b_dkv = (2 * nq + 2 * nk) * eb + 3 * rows + 2 * nk * eb      # ... in; dk, dv out
        out["fwd"].update(us=ms["fwd"] * 1e3, gbs=b_fwd / (ms["fwd"] * 1e-3) / 1e9)
        out["bwd"].update(us=ms_bwd * 1e3, gbs=(bytes_delta + b_dq + b_dkv) / (ms_bwd * 1e-3) / 1e9,
                          dq_gbs=b_dq / (ms["dq"] * 1e-3) / 1e9, dkv_gbs=b_dkv / (ms["dkv"] * 1e-3) / 1e9)
        out["note"] = "warm-cache latency: operands (2 MB) stay in L2 between launches"
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="cfg2", choices=["cfg1", "cfg2", "cfg3", "cfg4", "cfg5", "d256"])
    ap.add_argument("--only", action="store_true", help="measure the headline configuration only")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus must be 1 (sharding is design-only, B x Hkv across GPUs)")

    import torch
    from flex_attention_tpu_amd import configs

    name = "cfg2" if args.config == "cfg3" else args.config
    cfg = configs.CONFIGS.get(name) or configs.EXTRA_CONFIGS[name]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    r = measure(cfg, args.steps, args.warmup)
    head = summary(cfg, r)
    others = {}
    if not args.only:
        for other in ("cfg1", "cfg2", "cfg4", "cfg5", "d256"):
            if other != name:
                c = configs.CONFIGS.get(other) or configs.EXTRA_CONFIGS[other]
                others[other] = summary(c, measure(c, args.steps, args.warmup))
                torch.cuda.empty_cache()

    # A plain device copy of known size (256 MiB read + 256 MiB written per launch): the reference
    # dispatch that FETCH_SIZE / WRITE_SIZE counter readings of the attention kernels are scaled by.
    src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()

    ms = r["ms"]
    f_fwd = configs.flops_fwd(cfg)
    bf16 = r["elem_bytes"] == 2
    # roofline of the dominant kernel; algorithmic FLOPs of one launch:
    #   fwd 2 matmuls = F_fwd, dk/dv 4 matmuls = 2 F_fwd, dq 3 matmuls = 1.5 F_fwd (1 matmul from exchanged dS)
    algo = {"fwd": f_fwd, "dq": (0.5 if r["ds_used"] else 1.5) * f_fwd, "dkv": 2.0 * f_fwd}
    ms = dict(ms)
    if r["delta_fused"]:
        ms["dq"] = ms["dq_given_delta"]   # (the roofline object is about single kernels: the dq kernel without the delta kernel)
    dom = max(algo, key=lambda n: ms[n])
    traffic, stale = counter_traffic(dom) if name == "cfg2" else (None, None)
    roofline = {
        "kernel": dom, "bound": "mfma", "achieved": tf(algo[dom], ms[dom]), "peak": PEAK_BF16_TFLOPS,
        "unit": "TFLOP/s", "frac": tf(algo[dom], ms[dom]) / PEAK_BF16_TFLOPS,
        "traffic": traffic,
        "traffic_source": "profiles/bench_cfg2_hbm_traffic.txt (rocprofv3 --pmc runs of this script, not this run)"
                          if traffic is not None else None,
        "traffic_stale": stale,   # True: the kernel sources changed since the counter runs behind `traffic`
        "launch_ms": ms[dom], "launch_quantiles_ms": r["quantiles_ms"][dom],
    }
    if not bf16:
        b = head["bwd"]
        roofline.update(bound="hbm", achieved=b["dkv_gbs"], peak=PEAK_HBM_GBS, unit="GB/s", frac=b["dkv_gbs"] / PEAK_HBM_GBS)
    out = {
        "metric": "fwd & bwd attention TFLOP/s (S=4096,D=128,bf16 causal); % of MFMA peak",
        "value": head["step_tflops"],
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": r["ms_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if bf16 else "f32", "data": "synthetic",
        "config": {"workload": f"{cfg.name}{'+cfg3' if name == 'cfg2' else ''}: fwd + delta + dk/dv + dq, B={cfg.B} "
                               f"Hq={cfg.Hq} Hkv={cfg.Hkv} S={cfg.S} D={cfg.D} {'bf16' if bf16 else 'fp32'}, "
                               f"mask={cfg.mask}, score={cfg.score}, sm_scale=1/sqrt(D)"},
        "fwd": head["fwd"], "bwd": head["bwd"],
        "roofline": roofline,
        "other_configs": others,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
