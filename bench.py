#!/usr/bin/env python3
"""XFC step benchmark on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2] [--no-cpu]

A "step" is one pass of the hot path over one synthetic batch: fwd + loss
gradient (G), dX, dW fused with the SGD-momentum update of the fp16 label
matrix.  Inputs are resident in HBM before the timed region starts.  Prints ONE
JSON line.  The workload is BASELINE.json's headline configuration (configs[2]:
batch 512, d = 768, L = 1,310,720, fp16 storage, fp32 accumulate).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MFMA_F16_PEAK_TFLOPS = 2516.6   # MI355X dense fp16, AMD's published figure
HBM_PEAK_GBS = 8000.0           # MI355X HBM3E, AMD's published figure

# HBM bytes per launch of the dW+update kernel at configs[2]: rocprofv3 --pmc FETCH_SIZE (2,860,723.5 KiB,
# x2.000 from the 1 GiB copy) + WRITE_SIZE (3,932,160 KiB, x1.000); see profiles/xfc_step_cfg2_hbm_traffic_pmc.md.
DW_UPDATE_TRAFFIC_BYTES = {2: (2 * 2820425.4 + 3932160.0) * 1024.0}


def cpu_baseline(cfg: int, d: int, seed: int):
    """The CPU oracle (fp32 torch restatement of the reference's formulation) timed on this
    host's cores on a label slice of the same workload, scaled to the full label count."""
    import torch

    from oracle import xfc_oracle as O
    from renee_amd import synth

    c = synth.CONFIGS[cfg]
    B, L = c["B"], c["L"]
    Ls = min(L, 131072)
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    torch.set_num_threads(threads)
    X = synth.make_X(B, d, seed)
    W = synth.make_W(Ls, d, seed)
    M = torch.zeros_like(W)
    P = synth.make_positives(B, Ls, c["kmax"], c["kmean"], c["zipf"], seed)
    px, py = P.coo()
    times = []
    t_all = time.perf_counter()
    for i in range(8):
        t0 = time.perf_counter()
        r = O.step(X, W, M, px, py, 0.05, 0.9, 0.0, 1.0)
        W, M = r["W"], r["M"]
        times.append(time.perf_counter() - t0)
        if i >= 2 and time.perf_counter() - t_all > 25.0:
            break
    t = sorted(times[1:])[len(times[1:]) // 2]  # median, first step dropped
    t_full = t * (L / Ls)
    return {"value": B / t_full, "unit": "samples/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"B={B}, d={d}, label slice {Ls} of {L} (fp32 torch CPU ops, median of {len(times) - 1} steps "
                      f"= {t:.3f} s, scaled x{L / Ls:.0f} to the full label count)",
            "gflops": 6.0 * B * Ls * d / t / 1e9}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", type=int, default=2, help="index into BASELINE.json configs (1..4)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--calibrate", action="store_true",
                    help="after the timed region, run one 1 GiB xfc_copy (the known-size kernel the traffic "
                         "counters are scaled by when this command runs under rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (label sharding across GPUs is design-only); use --gpus 1",
              file=sys.stderr)
        return 2

    import torch

    from renee_amd import XFCLayer, synth

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    dev = torch.device("cuda:0")
    c = synth.CONFIGS[args.config]
    B, L, d = c["B"], c["L"], synth.D_MODEL
    layer = XFCLayer(L, d, B, dev, lr=0.05, momentum=0.9, weight_decay=0.0, seed=args.seed)
    X = synth.make_X(B, d, args.seed, dev).half()
    P = synth.make_positives(B, L, c["kmax"], c["kmean"], c["zipf"], args.seed)
    rowptr = torch.from_numpy(P.rowptr).to(dev)
    colidx = torch.from_numpy(P.colidx).to(dev)

    def step(ev=None):
        if ev:
            ev[0].record()
        layer.fwd_grad(X, rowptr=rowptr, colidx=colidx)
        if ev:
            ev[1].record()
        layer.dx(B, scale=1.0)
        if ev:
            ev[2].record()
        layer.dw_update(X)
        if ev:
            ev[3].record()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # events are recorded on torch's current stream, which is the stream every kernel is launched on
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(args.steps)]
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(evs[i])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    k_ms = [sum(e[i].elapsed_time(e[i + 1]) for e in evs) / args.steps for i in range(3)]
    gemm_flop = 2.0 * B * L * d
    step_tflops = 3 * gemm_flop / (ms_per_step * 1e-3) / 1e12
    upd_bytes = 8.0 * L * d  # read W, read M, write W, write M in fp16
    achieved = upd_bytes / (k_ms[2] * 1e-3) / 1e9
    out = {
        "metric": "XFC fwd+bwd+update samples/sec at d=768,L=1.31M fp16; % MFMA fp16 peak",
        "value": B / (ms_per_step * 1e-3),
        "unit": "samples/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"BASELINE configs[{args.config}]: XFC step, batch {B}, d={d}, L={L}, fp16 W/M/G, "
                               f"fp32 accumulate, {P.nnz} positives (Zipf s={c['zipf']})",
                   "batch": B, "d": d, "labels": L, "lr": 0.05, "momentum": 0.9},
        "step_tflops": step_tflops,
        "mfma_peak_frac": step_tflops / MFMA_F16_PEAK_TFLOPS,
        "kernels_ms": {"fwd_grad(+bucket)": k_ms[0], "dx(+reduce)": k_ms[1], "dw_update": k_ms[2]},
        "kernels_tflops": {"fwd_grad": gemm_flop / k_ms[0] / 1e9, "dx": gemm_flop / k_ms[1] / 1e9,
                           "dw_update": gemm_flop / k_ms[2] / 1e9},
        "roofline": {"kernel": "dw_kernel<DW_UPDATE> (dW GEMM + SGD-momentum update)", "bound": "hbm",
                     "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": DW_UPDATE_TRAFFIC_BYTES.get(args.config)},
    }
    if args.calibrate:
        from renee_amd._lib import check, lib

        src = torch.zeros(1 << 29, dtype=torch.float16, device=dev)  # 1 GiB
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        check(lib().xfc_copy(src.data_ptr(), dst.data_ptr(), src.numel() * 2,
                             torch.cuda.current_stream().cuda_stream), "xfc_copy")
        torch.cuda.synchronize()
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(args.config, d, args.seed)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
