#!/usr/bin/env python3
"""Benchmark of the fused gather-GEMM-scatter path on one MI355X.

Default workload (the one the headline metric is quoted on): the indoor-like
cloud of ~200 k voxels, 27 offsets, 64 -> 64 channels, fp16, one step =
forward + input gradient + weight gradient.  The protocol follows the
reference's timing script (warm-up calls, then timed calls back to back,
spconv-test.py:95-122) with longer defaults, 200 + 1000 steps instead of 10 + 100:
a step is 0.15 ms and the first few milliseconds after idle run about 8 % slower
(--warmup 10 --steps 100 reproduces the short protocol).

Prints ONE JSON line:  effective TFLOP/s = passes * 2 * M * Cin * Cout / t with
M the real (unpadded) pair count, a roofline object for the dominant kernel
(duration from HIP events on the launch stream) and the CPU baseline (the C
restatement of cpu-check.py / cpu-check-back.py on this box's host cores).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"f16": 2500.0, "f32": 157.3}      # dense MFMA: fp16 and bf16 alike, fp32
PEAK_HBM_GBS = 8000.0

WORKLOADS = {
    # name: (config id, variant, passes)
    "cfg2-indoor200k-k27-64x64-fp16-fwd+dgrad+wgrad": (2, "fp16", ("fwd", "dgrad", "wgrad")),
    "cfg2-indoor200k-k27-64x64-fp16-fwd": (2, "fp16", ("fwd",)),
    "cfg2-indoor200k-k27-64x64-fp32-fwd": (2, None, ("fwd",)),
    "cfg2-indoor200k-k27-64x64-tf32-fwd": (2, "tf32", ("fwd",)),
    "cfg2-indoor200k-k27-64x64-tf32-fwd+dgrad+wgrad": (2, "tf32", ("fwd", "dgrad", "wgrad")),
    "cfg2-indoor200k-k27-64x64-fp32-fwd+dgrad+wgrad": (2, None, ("fwd", "dgrad", "wgrad")),
    "cfg1-planes20k-k27-32x32-fp32-fwd+dgrad+wgrad": (1, None, ("fwd", "dgrad", "wgrad")),
    "cfg3-lidar120k-k27-128x128-fp16-fwd+dgrad+wgrad": (3, None, ("fwd", "dgrad", "wgrad")),
    "cfg4-down-k8-64x128-fp16-fwd+dgrad+wgrad": (4, None, ("fwd", "dgrad", "wgrad")),
    "cfg4-up-k8-128x64-fp16-fwd+dgrad+wgrad": (4, "up", ("fwd", "dgrad", "wgrad")),
    "cfg5-skinny-k27-4x32-fp16-fwd": (5, "skinny", ("fwd",)),
    "cfg5-skinny-k27-4x32-fp32-fwd": (5, "skinny-fp32", ("fwd",)),
    "cfg5-wide50k-k27-256x256-fp16-fwd": (5, "wide", ("fwd",)),
    "cfg5-wide50k-k27-256x256-fp32-fwd": (5, "wide-fp32", ("fwd",)),
}
DEFAULT = "cfg2-indoor200k-k27-64x64-fp16-fwd+dgrad+wgrad"


def make_case(name, scale=1.0):
    import numpy as np
    from fgms_amd import clouds
    cfg, variant, passes = WORKLOADS[name]
    arch80 = variant == "tf32"
    L = clouds.config_case(cfg, None if variant == "tf32" else variant, scale=scale)
    return L, passes, arch80


def dataflow_bytes(L, which):
    """Bytes one pass moves if every gathered row is read once per pair and every
    result row written once per pair (the pair-list dataflow), plus maps and
    weights: M*(Cin+Cout)*s + 8*M + K*Cin*Cout*s."""
    s = L["in_feats"].dtype.itemsize
    m = len(L["imap"])
    return m * (L["c_in"] + L["c_out"]) * s + 8 * m + L["k_vol"] * L["c_in"] * L["c_out"] * s


def compulsory_bytes(L):
    """Bytes a pass cannot avoid: every source and result row once, the maps, the weights:
    (N_in*Cin + N_out*Cout)*s + 8*M + K*Cin*Cout*s."""
    s = L["in_feats"].dtype.itemsize
    m = len(L["imap"])
    return (L["n_in"] * L["c_in"] + L["n_out"] * L["c_out"]) * s + 8 * m + L["k_vol"] * L["c_in"] * L["c_out"] * s


def cpu_baseline(name, budget_s=12.0):
    """Times the CPU oracle (OpenMP, this box's host cores) on a bounded sample of
    the same workload and returns effective TFLOP/s."""
    from oracle import fgms_oracle as oracle
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(16, os.cpu_count() or 1)
    threads = max(1, min(threads, oracle.max_threads() if oracle.max_threads() > 0 else threads))

    def run(scale, repeats=1):
        L, passes, _ = make_case(name, scale)
        args = (L["knnz"], L["imap"], L["omap"])
        t0 = time.perf_counter()
        for _ in range(repeats):
            if "fwd" in passes:
                oracle.c_fwd(L["in_feats"], L["kernel"], *args, L["n_out"], threads=threads)
            if "dgrad" in passes:
                oracle.c_dgrad(L["out_grad"], L["kernel"], *args, L["n_in"], threads=threads)
            if "wgrad" in passes:
                oracle.c_wgrad(L["in_feats"], L["out_grad"], *args, L["k_vol"], threads=threads)
        dt = time.perf_counter() - t0
        flops = repeats * len(passes) * 2.0 * len(L["imap"]) * L["c_in"] * L["c_out"]
        return dt, flops, L

    scale = 0.05
    dt, flops, L = run(scale)          # probe, then a sample sized to the budget
    want = min(1.0, scale * budget_s / max(dt, 1e-3))
    repeats = 1
    if want > 1.2 * scale:
        # the full cloud costs dt / scale per repeat; repeat it to fill the budget
        repeats = max(1, min(200, int(budget_s / max(dt / scale * want, 1e-3))))
        scale = want
        dt, flops, L = run(scale, repeats)
    return {
        "value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "sample": "%s at %.0f%% of the voxels (%d voxels, %d pairs), %d x one pass each of %s, %.1f s"
                  % (name.split("-")[0] + " cloud", scale * 100, L["n_in"], len(L["imap"]), repeats,
                     "+".join(WORKLOADS[name][2]), dt),
    }


def measured_traffic(workload, kernel):
    """HBM bytes per launch of `kernel` on `workload`, from the committed
    rocprofv3 FETCH_SIZE / WRITE_SIZE summary (profiles/hbm_traffic.json: KiB per
    dispatch and the factors a plain copy of known size calibrates them with).
    None when that workload / kernel was not profiled."""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            t = json.load(f)
        e = t["workloads"][workload][kernel.split("(")[0]]
        return (e["fetch_kib"] * t["fetch_factor"] + e["write_kib"] * t["write_factor"]) * 1024.0
    except (OSError, KeyError, ValueError):
        return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", default=DEFAULT, choices=sorted(WORKLOADS))
    ap.add_argument("--policy", type=int, default=0, help="0 auto, 1 generic kernels, 2 pair-stationary MFMA")
    ap.add_argument("--no-plan", action="store_true", help="do not pass a kernel-map plan")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--scale", type=float, default=1.0, help="voxel-count scale (1.0 = the named size)")
    ap.add_argument("--map-build", action="store_true",
                    help="also time the device kernel-map builder and the plan build on the headline cloud")
    ap.add_argument("--copy-calib", action="store_true",
                    help="also run plain 256 MiB device copies (for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus %d is not supported (every figure is "
              "the single-GPU throughput at the full shape)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    from fgms_amd import capi
    from tests.gpu_util import to_dev

    capi.lib()  # fails loudly if the HIP library is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    L, passes, arch80 = make_case(args.workload, args.scale)
    D = to_dev(L)
    capi.set_kernel_policy(args.policy)
    plan = None if args.no_plan else capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])
    dt = D["in_feats"].dtype
    out = torch.zeros(D["n_out"], D["c_out"], dtype=dt, device="cuda")
    gi = torch.zeros(D["n_in"], D["c_in"], dtype=dt, device="cuda")
    gw = torch.zeros_like(D["kernel"])
    m = len(L["imap"])
    flops_pass = 2.0 * m * L["c_in"] * L["c_out"]

    def step():
        if "fwd" in passes:
            capi.fusion_fwd(D["in_feats"], D["kernel"], 0, out, D["kpos"], None, D["imap"], D["omap"],
                            False, arch80, plan=plan)
        if "dgrad" in passes and "wgrad" in passes:
            # both gradients in one call, as the reference's fgms_bwd_cuda computes them
            capi.bwd(D["out_grad"], D["in_feats"], D["kernel"], 0, gi, gw, D["kpos"], None,
                     D["imap"], D["omap"], False, arch80, plan=plan)
        else:
            if "dgrad" in passes:
                capi.dgrad(D["out_grad"], D["kernel"], gi, D["kpos"], D["imap"], D["omap"], plan=plan)
            if "wgrad" in passes:
                capi.wgrad(D["in_feats"], D["out_grad"], gw, D["kpos"], D["imap"], D["omap"], plan=plan)

    if args.copy_calib:
        a_ = torch.ones(256 << 20, dtype=torch.uint8, device="cuda")
        b_ = torch.empty_like(a_)
        for _ in range(3):
            b_.copy_(a_)
        torch.cuda.synchronize()
        del a_, b_
    for _ in range(args.warmup):
        step()
    out.zero_(); gi.zero_(); gw.zero_()
    torch.cuda.synchronize()
    # the timed region: exactly K steps, nothing else on the stream
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()

    # the same K steps again with a HIP event pair around every kernel launch (recorded on
    # the launch stream by the library): per-kernel durations.  Kept out of the timed region
    # above because the ten event records per step cost 20-30 us of stream time themselves.
    capi.profile_reset()
    capi.profile_enable(True)
    prof_steps = min(args.steps, 200)
    tp0 = time.perf_counter()
    for _ in range(prof_steps):
        step()
    torch.cuda.synchronize()
    tp1 = time.perf_counter()
    capi.profile_enable(False)
    recs = capi.profile_records()
    capi.profile_reset()

    # gather-only pass over the rows the planned kernels read: the memory-side floor
    gather_floor = None
    if plan is not None and L["k_vol"] <= 64 and (L["c_in"] * D["in_feats"].element_size()) % 16 == 0 \
            and (L["c_out"] * D["in_feats"].element_size()) % 16 == 0:
        capi.profile_enable(True)
        for _ in range(20):
            if "fwd" in passes:
                capi.probe_gather(D["in_feats"], plan, for_dgrad=False)
            if "dgrad" in passes:
                capi.probe_gather(D["out_grad"], plan, for_dgrad=True)
        torch.cuda.synchronize()
        capi.profile_enable(False)
        pr = {}
        for name, ms in capi.profile_records():
            pr.setdefault(name, []).append(ms)
        capi.profile_reset()
        gather_floor = {k.replace("gather_probe_kernel", "").strip("()") + "_ms": sum(v[2:]) / len(v[2:])
                        for k, v in pr.items()}
        gather_floor["what"] = ("fgms_probe_gather: the same neighbour-table gathers as the planned kernel, "
                                "nothing else (no weights, MFMA, LDS or result rows), all wave slots in use")

    # the steps before the path: pair lists from coordinates, plan from pair lists
    map_build = None
    if args.map_build:
        import numpy as np
        from fgms_amd import clouds
        vox = torch.from_numpy(np.ascontiguousarray(clouds.indoor_cloud())).cuda()
        offs = clouds.offsets_cube(3)
        for _ in range(3):
            capi.build_kernel_map(vox, vox, offs)
        capi.profile_enable(True)
        torch.cuda.synchronize()
        tb = time.perf_counter()
        for _ in range(10):
            im_, om_, kn_, kp_ = capi.build_kernel_map(vox, vox, offs)
        torch.cuda.synchronize()
        t_map = (time.perf_counter() - tb) / 10
        capi.profile_enable(False)
        pr = {}
        for name, ms in capi.profile_records():
            pr.setdefault(name, []).append(ms)
        capi.profile_reset()
        tb = time.perf_counter()
        for _ in range(10):
            capi.Plan(kp_, im_, om_, vox.shape[0], vox.shape[0]).close()
        torch.cuda.synchronize()
        t_plan = (time.perf_counter() - tb) / 10
        nbytes = 2 * vox.numel() * 4 + 2 * im_.numel() * 4     # coordinates read, pair lists written
        k_ms = {k: sum(v) / len(v) for k, v in pr.items()}
        map_build = {"voxels": int(vox.shape[0]), "pairs": int(im_.numel()), "k_vol": 27,
                     "build_kernel_map_ms": t_map * 1e3, "kernels_ms": k_ms,
                     "algorithmic_GBs": nbytes / (sum(k_ms.values()) * 1e-3) / 1e9,
                     "plan_create_ms": t_plan * 1e3,
                     "note": "wall clock per call incl. temporary allocations and the one synchronisation; "
                             "algorithmic bytes = coordinates read + pair lists written"}

    ms_per_step = (t1 - t0) * 1e3 / args.steps
    value = len(passes) * flops_pass / (ms_per_step * 1e-3) / 1e12

    # per-kernel averages from the HIP events recorded on the launch stream
    per = {}
    for name, ms in recs:
        per.setdefault(name, []).append(ms)
    kernels = {k: {"launches": len(v), "avg_ms": sum(v) / len(v)} for k, v in per.items()}
    arith = "f16" if dt == torch.float16 else "f32"
    roofline = None
    if kernels:
        dom = max(kernels, key=lambda k: kernels[k]["avg_ms"] * kernels[k]["launches"])
        avg_s = kernels[dom]["avg_ms"] * 1e-3
        skinny = min(L["c_in"], L["c_out"]) <= 16
        if skinny:
            which = "dgrad" if "dgrad" in dom else "fwd"
            ach = dataflow_bytes(L, which) / avg_s / 1e9
            roofline = {"bound": "hbm", "kernel": dom, "achieved": ach, "peak": PEAK_HBM_GBS,
                        "unit": "GB/s", "frac": ach / PEAK_HBM_GBS, "traffic": measured_traffic(args.workload, dom),
                        "avg_kernel_ms": kernels[dom]["avg_ms"],
                        # `achieved` prices the launch as pair-list dataflow (a row per pair); a
                        # kernel that keeps rows on chip moves less and can exceed the peak by
                        # that count.  The same launch against the bytes no kernel can avoid:
                        "compulsory_bytes": compulsory_bytes(L),
                        "compulsory_GBs": compulsory_bytes(L) / avg_s / 1e9,
                        "compulsory_frac": compulsory_bytes(L) / avg_s / 1e9 / PEAK_HBM_GBS}
        else:
            # the backward call's single launch computes both gradients
            parts = ("dgrad", "wgrad") if dom.startswith("bwd_fused") else \
                (("dgrad",) if "dgrad" in dom else (("wgrad",) if "wgrad" in dom else ("fwd",)))
            # fp32 tensors in tf32 mode: every product is three bf16 MFMAs (hi*hi + hi*lo + lo*hi),
            # so the matrix pipes do three times the algorithmic flop, at the 16-bit rate
            factor, peak = (3, PEAK_TFLOPS["f16"]) if "bf16x3" in dom else (1, PEAK_TFLOPS[arith])
            ach = factor * len(parts) * flops_pass / avg_s / 1e12
            flow = sum(dataflow_bytes(L, w_) for w_ in parts)
            roofline = {"bound": "mfma", "kernel": dom, "achieved": ach, "peak": peak,
                        "unit": "TFLOP/s", "frac": ach / peak, "traffic": measured_traffic(args.workload, dom),
                        "mfma_flop_per_algorithmic_flop": factor,
                        "avg_kernel_ms": kernels[dom]["avg_ms"],
                        # the same launch priced as pair-list dataflow bytes against HBM
                        "passes_in_kernel": list(parts),
                        "dataflow_bytes": flow,
                        "dataflow_GBs": flow / avg_s / 1e9}

    line = {
        "metric": "effective TFLOP/s (2*sum|map_k|*Cin*Cout/t), %s, %s"
                  % ("+".join(passes), "tf32 mode" if arch80 else ("fp16" if arith == "f16" else "fp32")),
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "ms_per_step_with_kernel_events": (tp1 - tp0) * 1e3 / prof_steps,
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": arith, "data": "synthetic",
        "config": {"workload": args.workload, "voxels_in": L["n_in"], "voxels_out": L["n_out"],
                   "pairs": m, "k_vol": L["k_vol"], "c_in": L["c_in"], "c_out": L["c_out"],
                   "plan": plan is not None, "policy": args.policy,
                   "row_slots_per_pair": (round(plan.stats()["blocks_fwd"] * 64.0 / max(plan.stats()["pairs"], 1), 3)
                                          if plan is not None else None)},
        "kernels": kernels,
        "roofline": roofline,
        "gather_floor": gather_floor,
        "map_build": map_build,
        "cpu_baseline": None if args.no_cpu else cpu_baseline(args.workload),
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
