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

Order of a run: per-kernel event pass, plan / map-build timings and the second
surface first (they double as clock warm-up: a run that asks for few steps is
otherwise measured during the first milliseconds after idle), then the W warm-up
steps, then the timed region of exactly K steps, then the CPU baseline.

`value` is the step through the C ABI with an explicit plan built before the timed
region; what building the plan costs is in the same line (`plan`): its wall-clock
cost per call, the step time when it is paid once per 1 / 4 / 16 layer-steps (a
point cloud changes every iteration, a kernel map serves the handful of layers of
one resolution), and the step time without any plan.  `surface_backend` is the
same step through the python extension FGMS.backend (the reference's three
functions; plan found in its cache).
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
    the same workload and returns effective TFLOP/s, with all the threads the box
    grants and with one."""
    from oracle import fgms_oracle as oracle
    host_cores = os.cpu_count() or 1
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(16, host_cores)
    threads = max(1, min(threads, oracle.max_threads() if oracle.max_threads() > 0 else threads))
    all_threads = threads

    def run(scale, repeats=1, threads=all_threads):
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
        # two passes at the sample's size tell what a repeat costs (the small probe also pays for
        # the thread pool's start and first-touch page faults); then as many as fill the budget
        scale = want
        dt, flops, L = run(scale, 2)
        repeats = max(1, min(200, int(budget_s / max(dt / 2, 1e-3))))
        dt, flops, L = run(scale, repeats)
    # one thread, on a sample a sixteenth of that (about the same time again at most)
    dt1, flops1, L1 = run(max(scale / 16.0, 0.01), 1, threads=1)
    return {
        "value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "host_cores": host_cores, "threads": threads,
        "value_1_thread": flops1 / dt1 / 1e12,
        "sample_1_thread": "%d voxels, %d pairs, one pass each, %.1f s" % (L1["n_in"], len(L1["imap"]), dt1),
        "sample": "%s at %.0f%% of the voxels (%d voxels, %d pairs), %d x one pass each of %s, %.1f s"
                  % (name.split("-")[0] + " cloud", scale * 100, L["n_in"], len(L["imap"]), repeats,
                     "+".join(WORKLOADS[name][2]), dt),
    }


TRAFFIC_SOURCE = ("profiles/hbm_traffic.json: rocprofv3 FETCH_SIZE / WRITE_SIZE of an earlier profiled run of this "
                  "command (KiB per dispatch, scaled by a plain copy of known size); not measured by this run")


def to_dev(L):
    """The numpy layer on the GPU (kernel_nnz stays on the host, as the reference reads it there)."""
    import numpy as np
    import torch
    d = {}
    for k, v in L.items():
        d[k] = torch.from_numpy(v).cuda() if isinstance(v, np.ndarray) and k != "knnz" else v
    d["knnz_host"] = torch.from_numpy(L["knnz"].astype(np.int32))
    return d


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
                    help="also report the device kernel-map builder's kernels (the map and plan build costs are always reported)")
    ap.add_argument("--surface", default="cabi", choices=["cabi", "backend"],
                    help="what `value` times: the C ABI with an explicit plan (default) or the python "
                         "extension FGMS.backend (plan from its cache); the other one is reported next to it")
    ap.add_argument("--copy-calib", action="store_true",
                    help="also run plain 256 MiB device copies (for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--pin-weights", type=int, default=-1, choices=[-1, 0, 1],
                    help="1: promise the library that the weights do not change between calls (fgms_weights_pin: "
                         "it keeps its re-laid copies), 0: do not; default: 1 for forward-only workloads "
                         "(inference), 0 for training steps")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus %d is not supported (every figure is "
              "the single-GPU throughput at the full shape)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    from fgms_amd import capi
    import FGMS.backend as backend

    capi.lib()  # fails loudly if the HIP library is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    L, passes, arch80 = make_case(args.workload, args.scale)
    D = to_dev(L)
    capi.set_kernel_policy(args.policy)
    backend.fgms_set_kernel_policy(args.policy)
    backend.fgms_plan_cache(not args.no_plan)

    pinned = args.pin_weights == 1 or (args.pin_weights < 0 and tuple(passes) == ("fwd",))
    if pinned:
        capi.weights_pin(D["kernel"])
        backend.fgms_weights_pin(D["kernel"])

    def make_plan():
        return capi.Plan(D["kpos"], D["imap"], D["omap"], D["n_in"], D["n_out"])

    plan = None if args.no_plan else make_plan()
    dt = D["in_feats"].dtype
    out = torch.zeros(D["n_out"], D["c_out"], dtype=dt, device="cuda")
    gi = torch.zeros(D["n_in"], D["c_in"], dtype=dt, device="cuda")
    gw = torch.zeros_like(D["kernel"])
    m = len(L["imap"])
    flops_pass = 2.0 * m * L["c_in"] * L["c_out"]

    def step_cabi(plan=plan):
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

    qkpos = torch.zeros_like(D["kpos"])      # (accepted and ignored: tiles are derived from kpos)
    backend_ok = ("dgrad" in passes) == ("wgrad" in passes)     # the extension has the reference's three functions only

    def step_backend():
        if "fwd" in passes:
            backend.fgms_fusion_fwd_cuda(D["in_feats"], D["kernel"], 0, out, D["kpos"], qkpos, D["imap"], D["omap"],
                                         False, arch80)
        if "dgrad" in passes:
            backend.fgms_bwd_cuda(D["out_grad"], D["in_feats"], D["kernel"], 0, gi, gw, D["kpos"], qkpos,
                                  D["imap"], D["omap"], False, arch80)

    if args.surface == "backend" and not backend_ok:
        print("bench.py: FGMS.backend has no entry point for one gradient alone", file=sys.stderr)
        sys.exit(2)
    step = step_backend if args.surface == "backend" else step_cabi
    other = step_cabi if args.surface == "backend" else (step_backend if backend_ok else None)

    def timed(fn, n):
        torch.cuda.synchronize()
        a = time.perf_counter()
        for _ in range(n):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - a) * 1e3 / n

    if args.copy_calib:
        a_ = torch.ones(256 << 20, dtype=torch.uint8, device="cuda")
        b_ = torch.empty_like(a_)
        for _ in range(3):
            b_.copy_(a_)
        torch.cuda.synchronize()
        del a_, b_
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

    # the steps before the path: pair lists from coordinates (the indoor cloud's workloads), plan
    # from pair lists; the same step with no plan at all; the other surface
    import numpy as np
    from fgms_amd import clouds
    plan_cost = {}
    t_plan = None
    if not args.no_plan:
        for _ in range(3):
            make_plan().close()
        torch.cuda.synchronize()
        # the build is asynchronous: what it costs a step is the time it keeps the stream busy
        # (HIP events on the stream around the call); the wall clock of create + wait for its
        # findings + destroy is reported next to it
        evs = []
        for _ in range(10):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            pl = make_plan()
            e1.record()
            evs.append((e0, e1))
            pl.usable()
            pl.close()
        torch.cuda.synchronize()
        t_plan = sum(a.elapsed_time(b) for a, b in evs) / len(evs)
        tb = time.perf_counter()
        for _ in range(10):
            pl = make_plan()
            pl.usable()
            pl.close()
        torch.cuda.synchronize()
        plan_cost["plan_create_ms"] = t_plan
        plan_cost["plan_create_what"] = "stream time of one fgms_plan_create (HIP events around the call)"
        plan_cost["plan_create_wait_destroy_wall_ms"] = (time.perf_counter() - tb) / 10 * 1e3
    map_build = None
    cfg_id = WORKLOADS[args.workload][0]
    if cfg_id in (2, 5) and "wide" not in args.workload and args.scale == 1.0:
        vox = torch.from_numpy(np.ascontiguousarray(clouds.indoor_cloud())).cuda()
        offs = clouds.offsets_cube(3)
        for _ in range(3):
            capi.build_kernel_map(vox, vox, offs)
        capi.profile_enable(args.map_build)
        torch.cuda.synchronize()
        tb = time.perf_counter()
        for _ in range(10):
            im_, om_, kn_, kp_ = capi.build_kernel_map(vox, vox, offs)
        torch.cuda.synchronize()
        t_map = (time.perf_counter() - tb) / 10
        capi.profile_enable(False)
        plan_cost["build_kernel_map_ms"] = t_map * 1e3
        if args.map_build:
            pr = {}
            for name, ms in capi.profile_records():
                pr.setdefault(name, []).append(ms)
            capi.profile_reset()
            nbytes = 2 * vox.numel() * 4 + 2 * im_.numel() * 4     # coordinates read, pair lists written
            k_ms = {k: sum(v) / len(v) for k, v in pr.items()}
            map_build = {"voxels": int(vox.shape[0]), "pairs": int(im_.numel()), "k_vol": 27,
                         "build_kernel_map_ms": t_map * 1e3, "kernels_ms": k_ms,
                         "algorithmic_GBs": nbytes / (sum(k_ms.values()) * 1e-3) / 1e9,
                         "plan_create_ms": t_plan,
                         "note": "wall clock per call incl. temporary allocations and the one synchronisation; "
                                 "algorithmic bytes = coordinates read + pair lists written"}
        del vox, im_, om_
    if not args.no_plan and args.surface == "cabi":
        capi.set_kernel_policy(args.policy)
        n_np = max(5, min(50, args.steps))
        step_cabi(plan=None)
        plan_cost["no_plan_ms_per_step"] = timed(lambda: step_cabi(plan=None), n_np)
        capi.set_kernel_policy(args.policy)
    surface_other = None
    if other is not None:
        n_o = max(20, min(200, args.steps))
        for _ in range(5):
            other()
        surface_other = {"ms_per_step": timed(other, n_o), "steps": n_o}

    # per-kernel durations: steps with a HIP event pair around every kernel launch (recorded on
    # the launch stream by the library).  Kept out of the timed region below because the ten
    # event records per step cost 20-30 us of stream time themselves.  It is the last of the
    # measurement passes, right in front of the warm-up steps: the passes before it leave gaps
    # (host work, synchronisations) after which the clocks take some 10 ms of load to come back
    # up, more than the few warm-up steps a short run asks for (measured: 20 timed steps after 5
    # warm-up steps 137-141 us per step coming from such a gap, 130.5-132.7 us behind 100 and
    # more steps of load; 1000 timed steps 131 us).
    for _ in range(5):
        step()
    capi.profile_reset()
    capi.profile_enable(True)
    prof_steps = max(min(args.steps, 200), 100)
    tp0 = time.perf_counter()
    for _ in range(prof_steps):
        step()
    torch.cuda.synchronize()
    tp1 = time.perf_counter()
    capi.profile_enable(False)
    recs = capi.profile_records()
    capi.profile_reset()


    # W warm-up steps, then the timed region: exactly K steps, nothing else on the stream
    for _ in range(args.warmup):
        step()
    out.zero_(); gi.zero_(); gw.zero_()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()

    ms_per_step = (t1 - t0) * 1e3 / args.steps
    step_flops = len(passes) * flops_pass
    value = step_flops / (ms_per_step * 1e-3) / 1e12
    if t_plan is not None:
        # one plan build per `reuse` layer-steps (a layer-step = this workload's step)
        plan_cost["incl_plan"] = {
            "reuse_%d" % r: {"ms_per_step": ms_per_step + t_plan / r,
                             "value": step_flops / ((ms_per_step + t_plan / r) * 1e-3) / 1e12}
            for r in (1, 4, 16)}
    if "no_plan_ms_per_step" in plan_cost:
        plan_cost["no_plan_value"] = step_flops / (plan_cost["no_plan_ms_per_step"] * 1e-3) / 1e12
    if surface_other is not None:
        surface_other["value"] = step_flops / (surface_other["ms_per_step"] * 1e-3) / 1e12

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
            # HBM-bound launch: the algorithmic bytes are the ones no kernel can avoid (every
            # tensor once); a kernel that keeps result rows on chip moves fewer bytes than the
            # pair-list count (a row per pair), so that count is reported as a pricing only
            traffic = measured_traffic(args.workload, dom)
            ach = compulsory_bytes(L) / avg_s / 1e9
            roofline = {"bound": "hbm", "kernel": dom, "achieved": ach, "peak": PEAK_HBM_GBS,
                        "unit": "GB/s", "frac": ach / PEAK_HBM_GBS, "traffic": traffic,
                        "traffic_source": TRAFFIC_SOURCE if traffic is not None else None,
                        "traffic_GBs": traffic / avg_s / 1e9 if traffic is not None else None,
                        "avg_kernel_ms": kernels[dom]["avg_ms"],
                        "algorithmic_bytes": compulsory_bytes(L),
                        "algorithmic_bytes_what": "(N_in*Cin + N_out*Cout)*s + 8*M + K*Cin*Cout*s: every tensor once",
                        "pair_list_pricing_bytes": dataflow_bytes(L, which),
                        "pair_list_pricing_GBs": dataflow_bytes(L, which) / avg_s / 1e9}
        else:
            # the backward call's single launch computes both gradients
            parts = ("dgrad", "wgrad") if dom.startswith("bwd_fused") else \
                (("dgrad",) if "dgrad" in dom else (("wgrad",) if "wgrad" in dom else ("fwd",)))
            # fp32 tensors in tf32 mode: every product is three bf16 MFMAs (hi*hi + hi*lo + lo*hi),
            # so the matrix pipes do three times the algorithmic flop, at the 16-bit rate
            factor, peak = (3, PEAK_TFLOPS["f16"]) if "bf16x3" in dom else (1, PEAK_TFLOPS[arith])
            ach = factor * len(parts) * flops_pass / avg_s / 1e12
            flow = sum(dataflow_bytes(L, w_) for w_ in parts)
            traffic = measured_traffic(args.workload, dom)
            roofline = {"bound": "mfma", "kernel": dom, "achieved": ach, "peak": peak,
                        "unit": "TFLOP/s", "frac": ach / peak, "traffic": traffic,
                        "traffic_source": TRAFFIC_SOURCE if traffic is not None else None,
                        "mfma_flop_per_algorithmic_flop": factor,
                        # `frac` prices the matrix pipes' work (for split bf16: three MFMA flop per
                        # algorithmic flop); frac_algorithmic prices the useful work alone, against
                        # the same 16-bit peak and against the fp32 MFMA peak the tensors' type has
                        "frac_algorithmic": len(parts) * flops_pass / avg_s / 1e12 / peak,
                        "frac_algorithmic_of_fp32_peak": (len(parts) * flops_pass / avg_s / 1e12 / PEAK_TFLOPS["f32"]
                                                          if arith == "f32" else None),
                        "avg_kernel_ms": kernels[dom]["avg_ms"],
                        "passes_in_kernel": list(parts),
                        "algorithmic_flop": factor * len(parts) * flops_pass,
                        # the same launch PRICED as pair-list bytes (a gathered row and a result row
                        # per pair) -- a pricing, not traffic: caches serve the re-reads
                        "pair_list_pricing_bytes": flow,
                        "pair_list_pricing_GBs": flow / avg_s / 1e9}

    line = {
        "metric": "effective TFLOP/s (2*sum|map_k|*Cin*Cout/t), %s, %s"
                  % ("+".join(passes), "tf32 mode" if arch80 else ("fp16" if arith == "f16" else "fp32")),
        "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "ms_per_step_with_kernel_events": (tp1 - tp0) * 1e3 / prof_steps,
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": arith, "data": "synthetic",
        "config": {"workload": args.workload, "voxels_in": L["n_in"], "voxels_out": L["n_out"],
                   "pairs": m, "k_vol": L["k_vol"], "c_in": L["c_in"], "c_out": L["c_out"],
                   "plan": plan is not None, "policy": args.policy, "surface": args.surface,
                   "weights_pinned": pinned,
                   "row_slots_per_pair": (round(plan.stats()["blocks_fwd"] * 64.0 / max(plan.stats()["pairs"], 1), 3)
                                          if plan is not None else None)},
        "kernels": kernels,
        "roofline": roofline,
        "gather_floor": gather_floor,
        "plan": plan_cost or None,
        ("surface_backend" if args.surface == "cabi" else "surface_cabi"): surface_other,
        "map_build": map_build,
        "cpu_baseline": None if args.no_cpu else cpu_baseline(args.workload),
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
