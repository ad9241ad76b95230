#!/usr/bin/env python3
"""XFC step benchmark on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2] [--no-cpu] [--no-others]

A "step" is one pass of the hot path over one synthetic batch: fwd + loss
gradient (G), dX, dW fused with the SGD-momentum update of the fp16 label
matrix.  Inputs are resident in HBM before the timed region starts.  Prints ONE
JSON line.  The workload is BASELINE.json's headline configuration (configs[2]:
batch 512, d = 768, L = 1,310,720, fp16 storage, fp32 accumulate).

`ms_per_step` (and `value`) is wall-clock time over K steps run back to back between
two device synchronisations, starting from W ~ N(0, 0.02) as initialised and the
momentum left by the first step.  Beside it, `ms_per_step_events` gives the mean,
median and minimum of K per-step HIP event intervals measured with W and M put
back (xfc_copy) before each step, outside the step's event pair, so that every one
of those steps runs on the stated data (at lr = 0.05 W drifts from step to step);
the per-kernel times come from the same events.
The other BASELINE configurations (0 with a batch-256 run at the same label count
beside it, 1, 3 with its top-5 / top-100 scorers, 4) are timed the same way with
fewer steps and reported under `other_configs`;
`master_weights` times the update pass with fp32 master weights and momentum, and
`mfma_power_probe` runs the logits kernel on random and on all-zero operands.
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

# HBM bytes per launch of the dW+update kernel: rocprofv3 --pmc FETCH_SIZE (KiB, x2.000 from the 1 GiB
# copy in the same run) + WRITE_SIZE (KiB, x1.000); see profiles/xfc_step_cfg2_hbm_traffic_pmc.md.
DW_UPDATE_TRAFFIC_BYTES = {2: (2.000 * 2800162.7 + 1.000 * 3932160.0) * 1024.0,
                           # the other configurations: profiles/xfc_step_other_configs_hbm_traffic_pmc.md
                           1: (2.000 * 285086.0 + 1.000 * 393216.0) * 1024.0,
                           3: (2.000 * 8560528.2 + 1.000 * 8436843.0) * 1024.0,
                           4: (2.000 * 49418471.8 + 1.000 * 50331648.0) * 1024.0}


def _oracle_steps(B, L, d, c, seed, n_max, budget_s, warm):
    import torch

    from oracle import xfc_oracle as O
    from renee_amd import synth

    X = synth.make_X(B, d, seed)
    W = synth.make_W(L, d, seed)
    M = torch.zeros_like(W)
    P = synth.make_positives(B, L, c["kmax"], c["kmean"], c["zipf"], seed)
    px, py = P.coo()
    times = []
    t_all = time.perf_counter()
    for i in range(n_max):
        t0 = time.perf_counter()
        r = O.step(X, W, M, px, py, 0.05, 0.9, 0.0, 1.0)
        W, M = r["W"], r["M"]
        times.append(time.perf_counter() - t0)
        if i >= warm + 4 and time.perf_counter() - t_all > budget_s:
            break
    return sorted(times[warm:])


def cpu_baseline(cfg: int, d: int, seed: int):
    """The CPU oracle (fp32 torch restatement of the reference's formulation) timed on this
    host's cores on a label slice of the same workload, scaled to the full label count."""
    import torch

    from renee_amd import synth

    c = synth.CONFIGS[cfg]
    B, L = c["B"], c["L"]
    Ls = min(L, 131072)
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or (os.cpu_count() or 1)
    torch.set_num_threads(threads)
    ts = _oracle_steps(B, Ls, d, c, seed, 8, 20.0, 1)
    t = ts[len(ts) // 2]
    t_full = t * (L / Ls)
    return {"value": B / t_full, "unit": "samples/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"B={B}, d={d}, label slice {Ls} of {L} (fp32 torch CPU ops, median of {len(ts)} steps "
                      f"= {t:.3f} s, scaled x{L / Ls:.0f} to the full label count)",
            "gflops": 6.0 * B * Ls * d / t / 1e9}


def cpu_baseline_cfg0(d: int, seed: int):
    """BASELINE configs[0] as it stands: batch 32, L = 131,072, fp32, the whole step on the host's
    cores, 2 warm-up steps, median and minimum of at least 5 timed steps, nothing scaled."""
    import torch

    from renee_amd import synth

    c = synth.CONFIGS[0]
    B, L = c["B"], c["L"]
    ts = _oracle_steps(B, L, d, c, seed, 12, 10.0, 2)
    t = ts[len(ts) // 2]
    return {"value": B / t, "unit": "samples/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"BASELINE configs[0] unscaled: B={B}, d={d}, L={L}, fp32 torch CPU ops, 2 warm-up steps, "
                      f"median of {len(ts)} steps = {t:.4f} s (min {ts[0]:.4f} s)",
            "s_per_step_median": t, "s_per_step_min": ts[0], "gflops": 6.0 * B * L * d / t / 1e9}


def time_config(cfg: int, steps: int, warmup: int, seed: int, dev, wall_clock: bool = True, scorers: bool = False,
                batch: int = 0, loss_variant: bool = False, graph: bool = False):
    """Times `steps` steps of one BASELINE configuration (with `batch` rows instead of its own when
    given), each from the same (W0, M1) state."""
    import torch

    from renee_amd import XFCLayer, synth
    from renee_amd._lib import check, lib

    c = synth.CONFIGS[cfg]
    B, L, d = batch or c["B"], c["L"], synth.D_MODEL
    layer = XFCLayer(L, d, B, dev, lr=0.05, momentum=0.9, weight_decay=0.0, seed=seed)
    X = synth.make_X(B, d, seed, dev).half()
    P = synth.make_positives(B, L, c["kmax"], c["kmean"], c["zipf"], seed)
    rowptr = torch.from_numpy(P.rowptr).to(dev)
    colidx = torch.from_numpy(P.colidx).to(dev)
    h = lib()
    st = torch.cuda.current_stream().cuda_stream
    nbytes = L * d * 2

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

    # the state every timed step starts from: W as initialised, M as the first step leaves it
    W0 = layer.xfc_weight.clone()
    step()
    M1 = layer.momentum_buffer.clone()

    def restore():
        check(h.xfc_copy(W0.data_ptr(), layer.xfc_weight.data_ptr(), nbytes, st), "xfc_copy")
        check(h.xfc_copy(M1.data_ptr(), layer.momentum_buffer.data_ptr(), nbytes, st), "xfc_copy")

    for _ in range(warmup):
        restore()
        step()
    torch.cuda.synchronize()
    # events are recorded on torch's current stream, which is the stream every kernel is launched on
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        restore()
        step(evs[i])
    torch.cuda.synchronize()
    wall_with_restore = time.perf_counter() - t0
    per_step = sorted(e[0].elapsed_time(e[3]) for e in evs)
    ms_events = sum(per_step) / steps
    k_ms = [sum(e[i].elapsed_time(e[i + 1]) for e in evs) / steps for i in range(3)]
    out = {"B": B, "L": L, "d": d, "nnz": P.nnz, "zipf": c["zipf"], "ms_per_step": ms_events, "k_ms": k_ms,
           "ms_events": {"mean": ms_events, "median": per_step[steps // 2], "min": per_step[0]},
           "wall_s_incl_restore": wall_with_restore}
    if wall_clock:
        # the contract's figure: K steps back to back between two synchronisations, nothing else in between
        restore()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        out["wall_ms_per_step"] = (time.perf_counter() - t0) * 1e3 / steps
        # the plain copy kernel on the same buffers: what an HBM read + write stream reaches on this box
        restore()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        n = 6
        e0.record()
        for _ in range(n // 2):
            restore()
        e1.record()
        torch.cuda.synchronize()
        out["copy_gbs"] = 2.0 * nbytes * n / (e0.elapsed_time(e1) * 1e-3) / 1e9
        # the same step with the update left unfused (the split-accumulation path: dW written as fp32, then a
        # streaming SGD-momentum kernel over W, M and dW): what the fused epilogue is to be compared with, and what
        # a pure read-modify-write stream of the update's shape reaches on this box
        n = 5
        ev = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(n + 1)]
        for i in range(n + 1):  # the first one allocates the gradient and is not counted
            restore()
            layer.fwd_grad(X, rowptr=rowptr, colidx=colidx)
            layer.dx(B, scale=1.0)
            ev[i][0].record()
            layer.dw_accumulate(X)
            ev[i][1].record()
            layer.optimizer_step()
            ev[i][2].record()
        torch.cuda.synchronize()
        dw_ms = sum(e[0].elapsed_time(e[1]) for e in ev[1:]) / n
        upd_ms = sum(e[1].elapsed_time(e[2]) for e in ev[1:]) / n
        out["unfused_update"] = {"dw_fp32_out_ms": dw_ms, "sgd_momentum_ms": upd_ms,
                                 "sgd_momentum_gbs": 12.0 * L * d / (upd_ms * 1e-3) / 1e9,
                                 "note": "xfc_dw (beta 0) + xfc_sgd_momentum in place of the fused dw_update; the "
                                         "streaming kernel moves 12 bytes per weight (W and M read and written, "
                                         "fp32 dW read)"}
    if loss_variant:
        # the forward pass of the reference's one step in a hundred: the same kernel with the summed BCE loss,
        # timed inside whole steps like the figure it is compared with (a forward pass run back to back with
        # itself is 15-20 % slower than one that follows the HBM-bound update pass: the chip's power budget)
        loss = torch.zeros(1, device=dev, dtype=torch.float32)
        n = 5
        ev = [[torch.cuda.Event(enable_timing=True) for _ in range(2)] for _ in range(n + 1)]
        for i in range(n + 1):  # the first one warms the kernel up and is not counted
            restore()
            ev[i][0].record()
            layer.fwd_grad(X, rowptr=rowptr, colidx=colidx, loss_out=loss)
            ev[i][1].record()
            layer.dx(B, scale=1.0)
            layer.dw_update(X)
        torch.cuda.synchronize()
        out["fwd_grad_with_loss_ms"] = sum(e[0].elapsed_time(e[1]) for e in ev[1:]) / n
    if graph:
        # The same step captured once as a HIP graph (xfc_step_csr: the entry points enqueue on the caller's stream
        # and neither allocate nor synchronise) and replayed back to back: what a small batch costs when the host's
        # launch gaps between the five kernels are taken out.
        restore()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                layer.step_csr(X, rowptr, colidx)
        torch.cuda.current_stream().wait_stream(side)
        for _ in range(3):
            g.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            g.replay()
        e1.record()
        torch.cuda.synchronize()
        out["graph_replay_ms_per_step"] = e0.elapsed_time(e1) / steps
        del g
    if scorers:
        restore()
        for K in (5, 100):
            layer.topk(X, K)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            n = 3
            e0.record()
            for _ in range(n):
                layer.topk(X, K)
            e1.record()
            torch.cuda.synchronize()
            out[f"top{K}_ms"] = e0.elapsed_time(e1) / n
    del layer, W0, M1
    torch.cuda.empty_cache()
    return out


def mfma_power_probe(dev):
    """xfc_logits on cache-resident 4096 x 4096 x 8192 operands, once with random and once with all-zero
    inputs: the same kernel, instruction stream and memory traffic, so the ratio is what operand
    switching activity (power) costs the matrix pipes on this chip."""
    import torch

    from renee_amd import XFCLayer

    B, L, d = 4096, 4096, 8192
    out = {"shape": f"{B}x{L}x{d} fp16 logits, operands resident in the L2 / Infinity Cache"}
    lay = XFCLayer(L, d, B, dev)
    for name in ("random", "zeros"):
        if name == "zeros":
            lay.xfc_weight.zero_()
            X = torch.zeros(B, d, device=dev, dtype=torch.float16)
        else:
            X = (torch.randn(B, d, device=dev) * 0.05).half()
        for _ in range(3):
            lay.xfc_forward(X)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(20):
            lay.xfc_forward(X)
        e1.record()
        torch.cuda.synchronize()
        out[f"{name}_tflops"] = 2.0 * B * L * d / (e0.elapsed_time(e1) / 20 * 1e-3) / 1e12
    del lay
    torch.cuda.empty_cache()
    return out


def master_weights_update(cfg: int, seed: int, dev):
    """The dW + update pass in the reference's optimizer regime (fp32 master weights and momentum, fp16
    copy of W written by the same pass: 18 bytes per weight) at one configuration."""
    import torch

    from renee_amd import XFCLayer, synth

    c = synth.CONFIGS[cfg]
    B, L, d = c["B"], c["L"], synth.D_MODEL
    lay = XFCLayer(L, d, B, dev, lr=0.05, momentum=0.9, seed=seed, master_weights=True)
    X = synth.make_X(B, d, seed, dev).half()
    P = synth.make_positives(B, L, c["kmax"], c["kmean"], c["zipf"], seed)
    lay.fwd_grad(X, rowptr=torch.from_numpy(P.rowptr).to(dev), colidx=torch.from_numpy(P.colidx).to(dev))
    for _ in range(2):
        lay.dw_update(X, lr=0.0)   # lr 0: the weights stay on the stated distribution, the traffic is the same
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    n = 5
    e0.record()
    for _ in range(n):
        lay.dw_update(X, lr=0.0)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / n
    del lay
    torch.cuda.empty_cache()
    return {"dw_update_master_ms": ms, "bytes_per_weight": 18, "gbs": 18.0 * L * d / (ms * 1e-3) / 1e9,
            "hbm_frac": 18.0 * L * d / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS}


def summarise(r, cfg=None):
    """Per-configuration figures from time_config's result."""
    B, L, d = r["B"], r["L"], r["d"]
    gemm_flop = 2.0 * B * L * d
    ms = r["ms_per_step"]
    tf = 3 * gemm_flop / (ms * 1e-3) / 1e12
    s = {"workload": f"batch {B}, d={d}, L={L}, {r['nnz']} positives (Zipf s={r['zipf']})",
         "ms_per_step": ms, "samples_per_s": B / (ms * 1e-3), "step_tflops": tf,
         "mfma_peak_frac": tf / MFMA_F16_PEAK_TFLOPS,
         "kernels_ms": {"fwd_grad(+bucket)": r["k_ms"][0], "dx(+reduce)": r["k_ms"][1], "dw_update": r["k_ms"][2]},
         "w_update_gbs": 8.0 * L * d / (r["k_ms"][2] * 1e-3) / 1e9,
         "w_update_hbm_frac": 8.0 * L * d / (r["k_ms"][2] * 1e-3) / 1e9 / HBM_PEAK_GBS}
    if cfg in DW_UPDATE_TRAFFIC_BYTES:
        s["dw_update_traffic"] = DW_UPDATE_TRAFFIC_BYTES[cfg]
        s["dw_update_gbs_incl_measured_traffic"] = DW_UPDATE_TRAFFIC_BYTES[cfg] / (r["k_ms"][2] * 1e-3) / 1e9
    for k in ("wall_ms_per_step", "ms_events", "copy_gbs", "top5_ms", "top100_ms", "graph_replay_ms_per_step"):
        if k in r:
            s[k] = r[k]
    if "top5_ms" in r:
        s["top5_tflops"] = gemm_flop / (r["top5_ms"] * 1e-3) / 1e12
    return s


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", type=int, default=2, help="index into BASELINE.json configs (0..4)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--no-others", action="store_true", help="skip the other BASELINE configurations")
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

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    dev = torch.device("cuda:0")
    r = time_config(args.config, args.steps, args.warmup, args.seed, dev, loss_variant=True)
    s = summarise(r)
    B, L, d = r["B"], r["L"], r["d"]
    gemm_flop = 2.0 * B * L * d
    k_ms = r["k_ms"]
    upd_bytes = 8.0 * L * d  # read W, read M, write W, write M in fp16
    achieved = upd_bytes / (k_ms[2] * 1e-3) / 1e9
    traffic = DW_UPDATE_TRAFFIC_BYTES.get(args.config)
    wall_ms = r["wall_ms_per_step"]
    wall_tf = 3 * gemm_flop / (wall_ms * 1e-3) / 1e12
    out = {
        "metric": "XFC fwd+bwd+update samples/sec at d=768,L=1.31M fp16; % MFMA fp16 peak",
        "value": B / (wall_ms * 1e-3),
        "unit": "samples/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": wall_ms,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"BASELINE configs[{args.config}]: XFC step, batch {B}, d={d}, L={L}, fp16 W/M/G, "
                               f"fp32 accumulate, {r['nnz']} positives (Zipf s={r['zipf']})",
                   "batch": B, "d": d, "labels": L, "lr": 0.05, "momentum": 0.9,
                   "timed_state": "the K timed steps run back to back from W ~ N(0,0.02) as initialised and the "
                                  "momentum of step 1"},
        "timing": "ms_per_step / value: wall clock over the K steps between two device synchronisations; "
                  "ms_per_step_events and kernels_ms: per-step HIP event intervals on the launch stream with W and M "
                  "restored before each step outside the interval",
        "ms_per_step_events": r["ms_events"],
        "step_tflops": wall_tf,
        "mfma_peak_frac": wall_tf / MFMA_F16_PEAK_TFLOPS,
        "copy_gbs": r.get("copy_gbs"),
        "unfused_update": r.get("unfused_update"),
        "kernels_ms": s["kernels_ms"],
        "fwd_grad_with_loss_ms": r.get("fwd_grad_with_loss_ms"),
        "kernels_tflops": {"fwd_grad": gemm_flop / k_ms[0] / 1e9, "dx": gemm_flop / k_ms[1] / 1e9,
                           "dw_update": gemm_flop / k_ms[2] / 1e9},
        "roofline": {"kernel": "dw_kernel<DW_UPDATE> (dW GEMM + SGD-momentum update)", "bound": "hbm",
                     "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": traffic,
                     "achieved_incl_measured_traffic": None if traffic is None else traffic / (k_ms[2] * 1e-3) / 1e9,
                     "copy_kernel_gbs_same_run": r.get("copy_gbs")},
        # the two MFMA-bound kernels of the step, each against the dense fp16 matrix peak on 2*B*L*d flop
        "rooflines": [
            {"kernel": "fwd_kernel<FWD_GRAD> (logits GEMM + sigmoid - target epilogue, incl. the bucket pass)",
             "bound": "mfma", "achieved": gemm_flop / k_ms[0] / 1e9, "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
             "frac": gemm_flop / k_ms[0] / 1e9 / MFMA_F16_PEAK_TFLOPS},
            {"kernel": "dx_kernel (G . W over label slices, incl. the reduce of the partial sums)",
             "bound": "mfma", "achieved": gemm_flop / k_ms[1] / 1e9, "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
             "frac": gemm_flop / k_ms[1] / 1e9 / MFMA_F16_PEAK_TFLOPS}],
    }
    if args.calibrate:
        from renee_amd._lib import check, lib

        src = torch.zeros(1 << 29, dtype=torch.float16, device=dev)  # 1 GiB
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        check(lib().xfc_copy(src.data_ptr(), dst.data_ptr(), src.numel() * 2,
                             torch.cuda.current_stream().cuda_stream), "xfc_copy")
        torch.cuda.synchronize()
        del src, dst
    if not args.no_others:
        others = {}
        for cfg, n in ((0, 20), (1, 20), (3, 6), (4, 3)):
            if cfg == args.config:
                continue
            others[f"configs[{cfg}]"] = summarise(time_config(cfg, n, 2, args.seed, dev, wall_clock=False,
                                                              scorers=(cfg == 3), graph=(cfg in (0, 1))), cfg)
            others[f"configs[{cfg}]"]["steps"] = n
        # what the 64-row tiles buy at batch 32: the same label count at batch 256 (one full-height tile)
        b256 = time_config(0, 20, 2, args.seed, dev, wall_clock=False, batch=256)["ms_per_step"]
        others["configs[0]"]["batch256_same_labels_ms_per_step"] = b256
        others["configs[0]"]["vs_quarter_of_batch256"] = others["configs[0]"]["ms_per_step"] / (b256 / 4.0)
        out["other_configs"] = others
        out["master_weights"] = master_weights_update(args.config, args.seed, dev)
        out["mfma_power_probe"] = mfma_power_probe(dev)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(args.config, d, args.seed)
        out["cpu_baseline_cfg0"] = cpu_baseline_cfg0(d, args.seed)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
