"""Benchmark of the flex-attention hot path on one MI355X.

One step = one pass of the hot path over one batch of synthetic input resident in HBM:
forward (saving l, m), delta pre-pass, dq backward, dk/dv backward, at B=4, H=32, S=4096, D=128,
bf16, causal (benchmark configurations 2 and 3; pass --config cfg4 / cfg5 for the others).
Prints ONE JSON line: whole-step algorithmic TFLOP/s, per-pass TFLOP/s and fraction of the bf16
MFMA peak, a roofline object for the dominant kernel and the CPU oracle timed on the host cores.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X published dense bf16 MFMA peak
PEAK_HBM_GBS = 8000.0


# HBM bytes per launch on the default workload (cfg2), from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs of this script, each counter scaled by its reading for the 256 MiB device copy that
# main() ends with (FETCH_SIZE x 2.0, WRITE_SIZE x 1.0).  Counter-derived, not measured per run.
HBM_TRAFFIC_BYTES = {"fwd": 668476257, "dq": 689215371, "dkv": 944777858}


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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", default="cfg2", choices=["cfg2", "cfg3", "cfg4", "cfg5"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus must be 1 (sharding is design-only, B x Hkv across GPUs)")

    import torch
    import flex_attention_tpu_amd as F
    from flex_attention_tpu_amd import configs

    name = "cfg2" if args.config == "cfg3" else args.config
    cfg = configs.CONFIGS[name]
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    q, k, v, do = configs.make_inputs(cfg, dev)
    mf, bf = configs.mask_fns(cfg)
    sfn = configs.score_fn(cfg)
    sc, blk = cfg.sm_scale, cfg.block

    def fwd():
        return F._flex_attention_impl(q, k, v, None, None, True, False, sc, 1, blk, blk, blk, False, bf, mf, sfn)

    def step():
        o, l, m = fwd()
        d = F.compute_delta(o, do)
        dq = F.flex_attention_bwd_dq(q, k, v, None, None, l, m, o, do, d, block_b=1, block_q=blk, block_k_major=blk,
                                     block_k=blk, sm_scale=sc, debug=False, score_fn=sfn, mask_fn=mf, block_mask_fn=bf)
        dk, dv = F.flash_attention_bwd_dkv(k, v, q, None, None, l, m, d, do, block_b=1, block_q=blk, block_q_major=blk,
                                           block_k_major=blk, block_k=blk, sm_scale=sc, causal=False, debug=False,
                                           score_fn=sfn, mask_fn=mf, block_mask_fn=bf)
        return o, dq, dk, dv

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0

    # Per-kernel launch durations: K back-to-back launches of one kernel between two HIP events on
    # the launch stream (single launches bracketed by events carry several us of marker overhead).
    o, l, m = fwd()
    d = F.compute_delta(o, do)
    launches = {
        "fwd": fwd,
        "delta": lambda: F.compute_delta(o, do),
        "dq": lambda: F.flex_attention_bwd_dq(q, k, v, None, None, l, m, o, do, d, block_b=1, block_q=blk,
                                              block_k_major=blk, block_k=blk, sm_scale=sc, debug=False, score_fn=sfn,
                                              mask_fn=mf, block_mask_fn=bf),
        "dkv": lambda: F.flash_attention_bwd_dkv(k, v, q, None, None, l, m, d, do, block_b=1, block_q=blk,
                                                 block_q_major=blk, block_k_major=blk, block_k=blk, sm_scale=sc,
                                                 causal=False, debug=False, score_fn=sfn, mask_fn=mf, block_mask_fn=bf),
    }
    ms = {}
    for name_k, fn in launches.items():
        fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(args.steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        ms[name_k] = e0.elapsed_time(e1) / args.steps

    # A plain device copy of known size (256 MiB read + 256 MiB written per launch): the reference
    # dispatch that FETCH_SIZE / WRITE_SIZE counter readings of the attention kernels are scaled by.
    src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()

    ms_step = wall * 1e3 / args.steps
    f_fwd = configs.flops_fwd(cfg)
    f_bwd = 2.5 * f_fwd
    ms_bwd = ms["delta"] + ms["dq"] + ms["dkv"]
    tf = lambda fl, t_ms: fl / (t_ms * 1e-3) / 1e12
    bytes_delta = 2 * q.numel() * q.element_size() + 4 * cfg.B * cfg.Hq * cfg.S

    # roofline of the dominant kernel; algorithmic FLOPs of one launch:
    #   fwd 2 matmuls = F_fwd, dq 3 matmuls = 1.5 F_fwd, dk/dv 4 matmuls = 2 F_fwd
    algo = {"fwd": f_fwd, "dq": 1.5 * f_fwd, "dkv": 2.0 * f_fwd}
    dom = max(algo, key=lambda n: ms[n])
    roofline = {
        "kernel": dom, "bound": "mfma", "achieved": tf(algo[dom], ms[dom]), "peak": PEAK_BF16_TFLOPS,
        "unit": "TFLOP/s", "frac": tf(algo[dom], ms[dom]) / PEAK_BF16_TFLOPS,
        "traffic": HBM_TRAFFIC_BYTES.get(dom) if name == "cfg2" else None,
        "launch_ms": ms[dom],
    }
    out = {
        "metric": "fwd & bwd attention TFLOP/s (S=4096,D=128,bf16 causal); % of MFMA peak",
        "value": tf(f_fwd + f_bwd, ms_step),
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{cfg.name}+cfg3: fwd + delta + dq + dk/dv, B={cfg.B} Hq={cfg.Hq} Hkv={cfg.Hkv} "
                               f"S={cfg.S} D={cfg.D} bf16, mask={cfg.mask}, score={cfg.score}, sm_scale=1/sqrt(D)"},
        "fwd": {"ms": ms["fwd"], "tflops": tf(f_fwd, ms["fwd"]), "frac_of_peak": tf(f_fwd, ms["fwd"]) / PEAK_BF16_TFLOPS},
        "bwd": {"ms": ms_bwd, "tflops": tf(f_bwd, ms_bwd), "frac_of_peak": tf(f_bwd, ms_bwd) / PEAK_BF16_TFLOPS,
                "delta_ms": ms["delta"], "dq_ms": ms["dq"], "dkv_ms": ms["dkv"],
                "delta_gbs": bytes_delta / (ms["delta"] * 1e-3) / 1e9},
        "roofline": roofline,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
