"""Sequence-length sweep of the three attention kernels on one MI355X, written as roofline CSVs.

Counterpart of the reference's roofline generators (flex_attention_dq_bwd.py:651-753 ``roofline()``,
main.py:279-348) and of the files they wrote on a TPU (roofline_data_flex.csv: ``SeqLen, Time_Sec,
TFLOPs, Intensity``): batch 1, 8 heads, head dim 128, bf16, causal, S = 1k ... 256k, one row per
sequence length and pass.  FLOPs and bytes follow the reference's conventions: causal counts
S^2 / 2 pairs; forward 4 D per pair, dq 6 D, dk/dv 8 D; bytes = every operand and result moved once.

    python -m flex_attention_tpu_amd.roofline --out roofline_mi355x.csv [--max-seq 65536] [--plot roofline.png]
    python -m flex_attention_tpu_amd.roofline --from-csv roofline_mi355x.csv --plot roofline.png   # plot only, no GPU
"""
from __future__ import annotations

import argparse
import csv
import sys

PEAK_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0


def sweep(max_seq: int = 65536, min_seq: int = 1024, heads: int = 8, iters: int = 10, causal: bool = True, device="cuda:0"):
    """Rows (dict) of the sweep.  Every length up to 262144 runs the generated-stream kernels (their list cache holds
    4096 kv tiles of 64 rows resp. 2048 q tiles of 128); longer sequences would take the kernels with a compiled
    main loop."""
    import torch
    import flex_attention_tpu_amd as F
    from flex_attention_tpu_amd import masks

    D, B = 128, 1
    rows = []
    S = min_seq
    while S <= max_seq:
        g = torch.Generator(device="cpu").manual_seed(S)
        q, k, v, do = (torch.randn(B, heads, S, D, generator=g).to(torch.bfloat16).to(device) for _ in range(4))
        sc = D ** -0.5
        mf, bf = masks.make_causal_mask_fns(128, 128) if causal else (None, None)
        o, l, m = F._flex_attention_impl(q, k, v, None, None, True, False, sc, 1, 128, 128, 128, False, bf, mf, None)
        d = F.compute_delta(o, do)
        passes = {
            "fwd": lambda: F._flex_attention_impl(q, k, v, None, None, True, False, sc, 1, 128, 128, 128, False, bf, mf, None),
            "dq": lambda: F.flex_attention_bwd_dq(q, k, v, None, None, l, m, o, do, d, block_b=1, block_q=128,
                                                  block_k_major=128, block_k=128, sm_scale=sc, debug=False,
                                                  mask_fn=mf, block_mask_fn=bf),
            "dkv": lambda: F.flash_attention_bwd_dkv(k, v, q, None, None, l, m, d, do, block_b=1, block_q=128,
                                                     block_q_major=128, block_k_major=128, block_k=128, sm_scale=sc,
                                                     causal=False, debug=False, mask_fn=mf, block_mask_fn=bf),
        }
        pairs = B * heads * (S * S / 2.0 if causal else float(S) * S)
        t_bytes = B * heads * S * D * 2.0   # one bf16 [B, H, S, D] tensor
        r_bytes = B * heads * S * 4.0       # one fp32 [B, H, S] row vector
        work = {"fwd": (4.0 * D * pairs, 4 * t_bytes + 2 * r_bytes),            # q, k, v -> o, l, m
                "dq": (6.0 * D * pairs, 5 * t_bytes + 3 * r_bytes),             # q, k, v, do, l, m, delta -> dq
                "dkv": (8.0 * D * pairs, 6 * t_bytes + 3 * r_bytes)}            # ... -> dk, dv
        n = max(2, min(iters, int(2e11 / pairs) + 2))
        for name, fn in passes.items():
            fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(n):
                fn()
            e1.record()
            torch.cuda.synchronize()
            t = e0.elapsed_time(e1) * 1e-3 / n
            flops, nbytes = work[name]
            rows.append({"SeqLen": S, "Pass": name, "Time_Sec": t, "TFLOPs": flops / t / 1e12,
                         "Intensity": flops / nbytes, "FracOfPeak": flops / t / 1e12 / PEAK_TFLOPS})
            print(f"S={S:7d} {name:4s} {t * 1e3:10.3f} ms {flops / t / 1e12:8.1f} TFLOP/s  intensity {flops / nbytes:9.1f} FLOP/B",
                  file=sys.stderr, flush=True)
        del q, k, v, do, o, l, m, d
        torch.cuda.empty_cache()
        S *= 2
    return rows


def write_csv(rows, path):
    with open(path, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=["SeqLen", "Pass", "Time_Sec", "TFLOPs", "Intensity", "FracOfPeak"])
        w.writeheader()
        for r in rows:
            w.writerow(r)


def read_csv(path):
    """Rows of a CSV written by write_csv (numbers parsed back)."""
    with open(path, newline="") as f:
        return [{k: (v if k == "Pass" else (int(v) if k == "SeqLen" else float(v))) for k, v in r.items()}
                for r in csv.DictReader(f)]


def plot(rows, path):
    """Log-log roofline (memory slope and MFMA ceiling) with the measured points; needs matplotlib."""
    import matplotlib
    matplotlib.use("Agg")
    import matplotlib.pyplot as plt
    xs = [2.0 ** e for e in range(4, 18)]
    plt.figure(figsize=(7, 4.5))
    plt.loglog(xs, [min(PEAK_TFLOPS, x * PEAK_HBM_GBS / 1e3) for x in xs], "k-", label="MI355X roofline (8 TB/s, 2.5 PFLOP/s)")
    for name, mark in (("fwd", "o"), ("dq", "s"), ("dkv", "^")):
        pts = [r for r in rows if r["Pass"] == name]
        plt.loglog([r["Intensity"] for r in pts], [r["TFLOPs"] for r in pts], mark + "-", label=name)
    fwd = [r for r in rows if r["Pass"] == "fwd"]
    for r in (fwd[0], fwd[-1]) if fwd else ():
        plt.annotate(f"S={r['SeqLen']}", (r["Intensity"], r["TFLOPs"]), textcoords="offset points", xytext=(4, -12), fontsize=7)
    plt.xlabel("arithmetic intensity (FLOP / byte)")
    plt.ylabel("TFLOP/s")
    plt.title("flex attention on MI355X: bf16, causal, B=1, H=8, D=128, S = 1k ... 256k", fontsize=9)
    plt.legend()
    plt.grid(True, which="both", alpha=0.3)
    plt.tight_layout()
    plt.savefig(path, dpi=120)


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--out", default="roofline_mi355x.csv")
    ap.add_argument("--min-seq", type=int, default=1024)
    ap.add_argument("--max-seq", type=int, default=65536)
    ap.add_argument("--heads", type=int, default=8)
    ap.add_argument("--iters", type=int, default=10)
    ap.add_argument("--plot", default=None, help="also write a roofline plot (PNG; needs matplotlib)")
    ap.add_argument("--from-csv", default=None, help="plot the rows of this CSV instead of measuring (no GPU needed)")
    args = ap.parse_args()
    if args.from_csv:
        rows = read_csv(args.from_csv)
    else:
        rows = sweep(args.max_seq, args.min_seq, args.heads, args.iters)
        write_csv(rows, args.out)
    if args.plot:
        plot(rows, args.plot)


if __name__ == "__main__":
    main()
